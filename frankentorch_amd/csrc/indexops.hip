// Integer-exact kernels: index_select / embedding gather, argmax, head split/merge permute.
// Pure copies and comparisons; results are bit-for-bit those of the CPU reference.

#include <type_traits>

#include <cstdlib>

#include "common.hpp"

namespace {

constexpr int kWave = 64;
constexpr int kBlock = 256;
constexpr int64_t kMaxGrid = 2147483647LL;

// normalize_strict_index_value (crates/ft-kernel-cpu/src/lib.rs:20058-20090): finite, no
// fractional part beyond f64::EPSILON, non-negative, < dim_size. Returns -1 when invalid.
__device__ __forceinline__ int64_t strict_index(double v, int64_t dim_size) {
    if (!isfinite(v)) return -1;
    double t = trunc(v);
    if (fabs(v - t) > 2.220446049250313e-16) return -1;
    if (v < 0.0 || v >= 9.2233720368547758e18) return -1;
    int64_t i = (int64_t)v;
    if (i < 0 || i >= dim_size) return -1;
    return i;
}

// 64-bit minimum over all launches' invalid positions. An integer min does not depend on the
// order in which the updates land, so the reported position is the same on every run.
__device__ __forceinline__ void report_bad(int64_t *bad, int64_t pos) {
    if (bad) atomicMin(reinterpret_cast<unsigned long long *>(bad), (unsigned long long)pos);
}

template <typename T>
__global__ __launch_bounds__(kBlock) void index_select_kernel(const T *__restrict__ input, int64_t outer,
                                                              int64_t dim_size, int64_t inner,
                                                              const double *__restrict__ indices, int64_t num_indices,
                                                              T *__restrict__ out, int64_t *bad) {
    // One wavefront per gathered run of `inner` elements.
    const int64_t run = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
    if (run >= outer * num_indices) return;
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t o = run / num_indices, ii = run % num_indices;
    const int64_t idx = strict_index(indices[ii], dim_size);
    if (idx < 0) {
        if (lane == 0 && o == 0) report_bad(bad, ii);
        return;
    }
    const T *src = input + (o * dim_size + idx) * inner;
    T *dst = out + run * inner;
    constexpr int EPV = 16 / sizeof(T);
    using V = typename std::conditional<sizeof(T) == 4, float4, double2>::type;
    if (inner % EPV == 0 && ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) == 0) {
        const int64_t nvec = inner / EPV;
        for (int64_t v = lane; v < nvec; v += kWave) reinterpret_cast<V *>(dst)[v] = reinterpret_cast<const V *>(src)[v];
    } else {
        for (int64_t j = lane; j < inner; j += kWave) dst[j] = src[j];
    }
}

__global__ __launch_bounds__(kBlock) void embedding_add_kernel(const float *__restrict__ wte, int64_t vocab,
                                                               const float *__restrict__ wpe,
                                                               const double *__restrict__ ids, int64_t tokens,
                                                               int64_t seq, int64_t width, float *__restrict__ out,
                                                               int64_t *bad) {
    const int64_t t = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
    if (t >= tokens) return;
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t idx = strict_index(ids[t], vocab);
    if (idx < 0) {
        if (lane == 0) report_bad(bad, t);
        return;
    }
    const float *a = wte + idx * width;
    const float *b = wpe + (t % seq) * width;
    float *dst = out + t * width;
    if (width % 4 == 0 &&
        ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(dst)) & 15u) == 0) {
        for (int64_t v = lane; v < width / 4; v += kWave) {
            float4 x = reinterpret_cast<const float4 *>(a)[v];
            float4 y = reinterpret_cast<const float4 *>(b)[v];
            reinterpret_cast<float4 *>(dst)[v] = make_float4(x.x + y.x, x.y + y.y, x.z + y.z, x.w + y.w);
        }
    } else {
        for (int64_t j = lane; j < width; j += kWave) dst[j] = a[j] + b[j];
    }
}

__global__ void set_i64_kernel(int64_t *p, int64_t v) { *p = v; }
// An index that failed validation was recorded as an unsigned minimum; "none" is all ones == -1.

// The reduced tensor is read once: non-temporal 128-bit loads (measured +2-8 % on streams that do not fit the caches).
typedef float nat_f4 __attribute__((ext_vector_type(4)));
typedef double nat_d2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float4 stream_load(const float4 *p) {
    nat_f4 v = __builtin_nontemporal_load(reinterpret_cast<const nat_f4 *>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ double2 stream_load(const double2 *p) {
    nat_d2 v = __builtin_nontemporal_load(reinterpret_cast<const nat_d2 *>(p));
    return make_double2(v.x, v.y);
}

// ---- argmax ----------------------------------------------------------------------------------
// Candidate = (value, first index reaching it) plus the first NaN position. Combining two
// candidates keeps the larger value, the smaller index on equal values, and the smaller NaN
// position: associative and commutative, so the tree shape cannot change the answer, and the
// answer equals the sequential scan of crates/ft-kernel-cpu/src/lib.rs:39518-39535
// (first strict maximum wins; the first NaN wins and ends the scan; all -inf gives index 0).
template <typename T> struct Cand {
    T val;
    int64_t idx;
    int64_t nan_idx;
};
constexpr int64_t kNoNan = 0x7fffffffffffffffLL;

template <typename T> __device__ __forceinline__ Cand<T> cand_init() {
    return Cand<T>{sizeof(T) == 4 ? (T)-__builtin_inff() : (T)-__builtin_inf(), 0, kNoNan};
}
template <typename T> __device__ __forceinline__ void cand_feed(Cand<T> &c, T v, int64_t i) {
    if (v != v) {
        if (i < c.nan_idx) c.nan_idx = i;
    } else if (v > c.val) {
        c.val = v;
        c.idx = i;
    }
}
template <typename T> __device__ __forceinline__ Cand<T> cand_merge(const Cand<T> &a, const Cand<T> &b) {
    Cand<T> r;
    if (b.val > a.val || (b.val == a.val && b.idx < a.idx)) {
        r.val = b.val;
        r.idx = b.idx;
    } else {
        r.val = a.val;
        r.idx = a.idx;
    }
    r.nan_idx = a.nan_idx < b.nan_idx ? a.nan_idx : b.nan_idx;
    return r;
}
template <typename T> __device__ __forceinline__ Cand<T> cand_shfl_xor(const Cand<T> &c, int off) {
    Cand<T> r;
    r.val = __shfl_xor(c.val, off, kWave);
    r.idx = __shfl_xor(c.idx, off, kWave);
    r.nan_idx = __shfl_xor(c.nan_idx, off, kWave);
    return r;
}

// Last-dim argmax: one block per row. Rows such as 50 257 floats start at arbitrary 4-byte offsets, so a row is read as a
// scalar head up to the first 16-byte boundary, 128-bit vectors, and a scalar tail. Every lane feeds its candidates in
// increasing index order (head < body < tail, and a lane's vectors ascend), which is what "first strict maximum" needs.
template <typename T>
__global__ __launch_bounds__(kBlock) void argmax_lastdim_kernel(const T *__restrict__ x, int64_t rows, int64_t cols,
                                                                T *__restrict__ out) {
    constexpr int EPV = 16 / (int)sizeof(T);
    using V = typename std::conditional<sizeof(T) == 4, float4, double2>::type;
    __shared__ Cand<T> smem[kBlock / kWave];
    const T *xr = x + (int64_t)blockIdx.x * cols;
    Cand<T> c = cand_init<T>();
    int64_t lead = (int64_t)(((16u - (unsigned)(reinterpret_cast<uintptr_t>(xr) & 15u)) & 15u) / sizeof(T));
    if (lead > cols) lead = cols;
    if ((int64_t)threadIdx.x < lead) cand_feed(c, xr[threadIdx.x], (int64_t)threadIdx.x);
    const int64_t nvec = (cols - lead) / EPV;
    const V *xv = reinterpret_cast<const V *>(xr + lead);
    auto feed_vec = [&](const V &v, int64_t vi) __attribute__((always_inline)) {
        const int64_t i0 = lead + vi * EPV;
        if constexpr (sizeof(T) == 4) {
            cand_feed(c, (T)v.x, i0);
            cand_feed(c, (T)v.y, i0 + 1);
            cand_feed(c, (T)v.z, i0 + 2);
            cand_feed(c, (T)v.w, i0 + 3);
        } else {
            cand_feed(c, (T)v.x, i0);
            cand_feed(c, (T)v.y, i0 + 1);
        }
    };
    int64_t j = threadIdx.x;
    // Eight independent 128-bit loads in flight per lane.
    for (; j + 7 * kBlock < nvec; j += 8 * kBlock) {
        V v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = stream_load(xv + j + u * kBlock);
#pragma unroll
        for (int u = 0; u < 8; ++u) feed_vec(v[u], j + u * kBlock);
    }
    for (; j < nvec; j += kBlock) feed_vec(stream_load(xv + j), j);
    const int64_t t0 = lead + nvec * EPV + threadIdx.x;
    if (t0 < cols) cand_feed(c, xr[t0], t0);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) c = cand_merge(c, cand_shfl_xor(c, off));
    if ((threadIdx.x & (kWave - 1)) == 0) smem[threadIdx.x / kWave] = c;
    __syncthreads();
    if (threadIdx.x == 0) {
        Cand<T> r = smem[0];
#pragma unroll
        for (int w = 1; w < kBlock / kWave; ++w) r = cand_merge(r, smem[w]);
        out[blockIdx.x] = (T)(r.nan_idx != kNoNan ? r.nan_idx : r.idx);
    }
}

// ---- argmax from the row maxima of column groups ----------------------------------------------
// gmax[g * rows + row] is the maximum of row `row` over columns [64 g, 64 g + 64), written by the product that made the
// logits, or NaN where that is not known (the group holds a NaN). A row's
// argmax is then the first element equal to the largest group maximum, in the first group that attains it -- found by
// reading that one group -- after the unknown groups have been scanned element by element with the rule of
// argmax_lastdim_kernel (first strict maximum; the first NaN wins), whose answer this reproduces bit for bit: a known group
// holds no NaN, its maximum is an element of it, and ties go to the earlier column either way. A workgroup takes 32
// consecutive rows (their group maxima are one 128-byte segment) and deals the groups, in column order, to 32 slices whose
// candidates are merged in that order.
constexpr int kGroupCols = 64;
constexpr int kGroupRows = 32;    // rows per workgroup: one per lane of a half wavefront
constexpr int kGroupSlices = 32;  // column slices per workgroup (1024 threads)
__global__ __launch_bounds__(kGroupRows * kGroupSlices) void argmax_group_kernel(const float *__restrict__ logits, int64_t rows, int64_t cols,
                                                                                  const float *__restrict__ gmax, int groups,
                                                                                  float *__restrict__ out) {
    __shared__ float s_val[kGroupSlices][kGroupRows];
    __shared__ int64_t s_idx[kGroupSlices][kGroupRows], s_nan[kGroupSlices][kGroupRows];
    __shared__ int s_grp[kGroupSlices][kGroupRows];
    const int lr = threadIdx.x % kGroupRows, slice = threadIdx.x / kGroupRows;
    const int64_t row = (int64_t)blockIdx.x * kGroupRows + lr;
    const bool live = row < rows;
    const int per = (groups + kGroupSlices - 1) / kGroupSlices;
    const int g0 = slice * per, g1 = g0 + per < groups ? g0 + per : groups;
    float val = -__builtin_inff();
    int64_t idx = 0, nan_idx = kNoNan;
    int grp = -1;  // >= 0: idx is only the group's first column, the element is still to be found
    const float *xr = logits + (live ? row : 0) * cols;
    if (live) {
        constexpr int kBatch = 8;  // group maxima fetched together: the loop is bound by memory latency, not by its arithmetic
        for (int gb = g0; gb < g1; gb += kBatch) {
            float mv[kBatch];
#pragma unroll
            for (int q = 0; q < kBatch; ++q) mv[q] = gb + q < g1 ? gmax[(int64_t)(gb + q) * rows + row] : -__builtin_inff();
#pragma unroll
            for (int q = 0; q < kBatch; ++q) {
                const float m = mv[q];
                const int g = gb + q;
                if (m != m) {
                    const int64_t c0 = (int64_t)g * kGroupCols, c1 = c0 + kGroupCols < cols ? c0 + kGroupCols : cols;
                    for (int64_t c = c0; c < c1; ++c) {
                        const float v = xr[c];
                        if (v != v) {
                            if (c < nan_idx) nan_idx = c;
                        } else if (v > val) {
                            val = v;
                            idx = c;
                            grp = -1;
                        }
                    }
                } else if (m > val) {
                    val = m;
                    idx = (int64_t)g * kGroupCols;
                    grp = g;
                }
            }
        }
    }
    s_val[slice][lr] = val;
    s_idx[slice][lr] = idx;
    s_nan[slice][lr] = nan_idx;
    s_grp[slice][lr] = grp;
    __syncthreads();
    if (slice != 0 || !live) return;
    for (int sl = 1; sl < kGroupSlices; ++sl) {  // column order: a later slice wins only with a strictly larger value
        if (s_val[sl][lr] > val) {
            val = s_val[sl][lr];
            idx = s_idx[sl][lr];
            grp = s_grp[sl][lr];
        }
        if (s_nan[sl][lr] < nan_idx) nan_idx = s_nan[sl][lr];
    }
    if (nan_idx != kNoNan) {
        idx = nan_idx;
    } else if (grp >= 0) {
        const int64_t c0 = (int64_t)grp * kGroupCols, c1 = c0 + kGroupCols < cols ? c0 + kGroupCols : cols;
        for (int64_t c = c0; c < c1; ++c)
            if (xr[c] == val) {
                idx = c;
                break;
            }
    }
    out[row] = (float)idx;
}

// Strided argmax over [outer, reduce, inner], inner > 1: one thread per output, coalesced on inner.
template <typename T>
__global__ __launch_bounds__(kBlock) void argmax_strided_kernel(const T *__restrict__ x, int64_t outer, int64_t reduce,
                                                                int64_t inner, T *__restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= outer * inner) return;
    const int64_t o = i / inner, in = i % inner;
    const T *xb = x + o * reduce * inner + in;
    Cand<T> c = cand_init<T>();
    for (int64_t r = 0; r < reduce; ++r) {
        T v = xb[r * inner];
        if (v != v) {
            c.nan_idx = r;
            break;
        }
        if (v > c.val) {
            c.val = v;
            c.idx = r;
        }
    }
    out[i] = (T)(c.nan_idx != kNoNan ? c.nan_idx : c.idx);
}

// ---- permute [d0, d1, d2, d3] -> [d0, d2, d1, d3] ------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kBlock) void permute_0213_kernel(const T *__restrict__ src, T *__restrict__ dst,
                                                              int64_t d0, int64_t d1, int64_t d2, int64_t d3,
                                                              int vec) {
    // One thread per `vec`-element chunk of the destination.
    const int64_t chunks_per_run = d3 / vec;
    const int64_t total = d0 * d1 * d2 * chunks_per_run;
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const int64_t c = i % chunks_per_run;
    int64_t t = i / chunks_per_run;
    const int64_t i1 = t % d1;  // destination order: [d0][d2][d1][d3]
    t /= d1;
    const int64_t i2 = t % d2;
    const int64_t i0 = t / d2;
    const T *s = src + (((i0 * d1 + i1) * d2 + i2) * d3) + c * vec;
    T *d = dst + (((i0 * d2 + i2) * d1 + i1) * d3) + c * vec;
    if (vec == 1) {
        *d = *s;
    } else {
        using V = typename std::conditional<sizeof(T) == 4, float4, double2>::type;
        *reinterpret_cast<V *>(d) = *reinterpret_cast<const V *>(s);
    }
}

// ---- batched 2-D transpose: dst[b][c][r] = src[b][r][c] -------------------------------------------
// A 64 x 64 tile goes through LDS so that both sides move whole 128-bit vectors along their contiguous dimension: a
// lane reads four consecutive columns of one source row and writes four consecutive rows' worth of one destination row.
// The tile is kept [column][row + pad]: the vector of a source row lands as four scalars 65 words apart (conflict-free
// over the 16 lanes of a row), and a destination row is read back as four consecutive words.
template <typename T>
__global__ __launch_bounds__(kBlock) void transpose_tile_kernel(const T *__restrict__ src, T *__restrict__ dst, int64_t rows,
                                                                int64_t cols, int64_t tiles_x) {
    constexpr int TS = 64, EPV = 16 / (int)sizeof(T), VPR = TS / EPV;  // vectors per tile row: 16 (fp32) or 32 (fp64)
    using V = typename std::conditional<sizeof(T) == 4, float4, double2>::type;
    __shared__ T tile[TS][TS + 1];
    const int64_t plane = rows * cols;
    const T *sp = src + (int64_t)blockIdx.y * plane;
    T *dp = dst + (int64_t)blockIdx.y * plane;
    const int64_t r0 = ((int64_t)blockIdx.x / tiles_x) * TS, c0 = ((int64_t)blockIdx.x % tiles_x) * TS;
    const int vx = threadIdx.x % VPR, vy = threadIdx.x / VPR;
    constexpr int RPP = kBlock / VPR;  // tile rows covered per pass
#pragma unroll
    for (int p = 0; p < TS / RPP; ++p) {
        const int r = vy + p * RPP;
        if (r0 + r < rows && c0 + vx * EPV < cols) {
            const V v = *reinterpret_cast<const V *>(sp + (r0 + r) * cols + c0 + vx * EPV);
            const T *e = reinterpret_cast<const T *>(&v);
#pragma unroll
            for (int j = 0; j < EPV; ++j) tile[vx * EPV + j][r] = e[j];
        }
    }
    __syncthreads();
#pragma unroll
    for (int p = 0; p < TS / RPP; ++p) {
        const int c = vy + p * RPP;
        if (c0 + c < cols && r0 + vx * EPV < rows) {
            V v;
            T *e = reinterpret_cast<T *>(&v);
#pragma unroll
            for (int j = 0; j < EPV; ++j) e[j] = tile[c][vx * EPV + j];
            *reinterpret_cast<V *>(dp + (c0 + c) * rows + r0 + vx * EPV) = v;
        }
    }
}

// Any extents and alignments: 32 x 32 tiles of single elements, both sides coalesced.
template <typename T>
__global__ __launch_bounds__(kBlock) void transpose_scalar_kernel(const T *__restrict__ src, T *__restrict__ dst, int64_t rows,
                                                                  int64_t cols, int64_t tiles_x) {
    __shared__ T tile[32][33];
    const int64_t plane = rows * cols;
    const T *sp = src + (int64_t)blockIdx.y * plane;
    T *dp = dst + (int64_t)blockIdx.y * plane;
    const int64_t r0 = ((int64_t)blockIdx.x / tiles_x) * 32, c0 = ((int64_t)blockIdx.x % tiles_x) * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int64_t r = r0 + ty + 8 * k, c = c0 + tx;
        if (r < rows && c < cols) tile[ty + 8 * k][tx] = sp[r * cols + c];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int64_t c = c0 + ty + 8 * k, r = r0 + tx;
        if (r < rows && c < cols) dp[c * rows + r] = tile[tx][ty + 8 * k];
    }
}

template <typename T>
int32_t launch_index_select(const T *input, int64_t outer, int64_t dim_size, int64_t inner, const double *indices,
                            int64_t num_indices, T *out, int64_t *bad, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(outer >= 0 && dim_size >= 0 && inner >= 0 && num_indices >= 0, "index_select: negative extent");
    hipStream_t st = fth::resolve_stream(s);
    if (bad) {
        set_i64_kernel<<<1, 1, 0, st>>>(bad, -1);
        FTH_CHECK_LAUNCH("index_select(bad_index reset)");
    }
    if (outer == 0 || inner == 0 || num_indices == 0) return FTH_OK;
    FTH_ARG(input && indices && out, "index_select: NULL operand");
    int64_t grid = fth::ceil_div(outer * num_indices, kBlock / kWave);
    FTH_ARG(grid <= kMaxGrid, "index_select: too many rows for one launch");
    index_select_kernel<T><<<dim3((unsigned)grid), dim3(kBlock), 0, st>>>(input, outer, dim_size, inner, indices,
                                                                           num_indices, out, bad);
    FTH_CHECK_LAUNCH("index_select");
    return FTH_OK;
}

template <typename T>
int32_t launch_argmax(const T *x, int64_t outer, int64_t reduce, int64_t inner, T *out, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(outer >= 0 && reduce >= 0 && inner >= 0, "argmax: negative extent");
    if (outer == 0 || inner == 0) return FTH_OK;
    if (reduce == 0) {
        fth::set_error(FTH_ERR_EMPTY_REDUCTION_DIM, "argmax over an empty dimension");
        fth::last_error().a = 0;
        return FTH_ERR_EMPTY_REDUCTION_DIM;
    }
    FTH_ARG(x && out, "argmax: NULL operand");
    hipStream_t st = fth::resolve_stream(s);
    if (inner == 1) {
        FTH_ARG(outer <= kMaxGrid, "argmax: too many rows for one launch");
        {
            // Long rows: three workgroups per compute unit, each lane with eight 128-bit loads in flight, read the stream
            // fastest (fp32 [8192, 50257]: eight per unit 0.770 of the HBM peak, four 0.806, three 0.823, two 0.700). The
            // kernel's registers would allow eight, so 48 KiB of unused dynamic LDS per workgroup hold the count at three.
            const size_t pad = reduce >= 8192 ? (size_t)48 * 1024 : 0;
            argmax_lastdim_kernel<T><<<dim3((unsigned)outer), dim3(kBlock), pad, st>>>(x, outer, reduce, out);
        }
    } else {
        int64_t grid = fth::ceil_div(outer * inner, kBlock);
        FTH_ARG(grid <= kMaxGrid, "argmax: too many lanes for one launch");
        argmax_strided_kernel<T><<<dim3((unsigned)grid), dim3(kBlock), 0, st>>>(x, outer, reduce, inner, out);
    }
    FTH_CHECK_LAUNCH("argmax");
    return FTH_OK;
}

template <typename T>
int32_t launch_permute(const T *src, T *dst, int64_t d0, int64_t d1, int64_t d2, int64_t d3, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(d0 >= 0 && d1 >= 0 && d2 >= 0 && d3 >= 0, "permute: negative extent");
    if (d0 == 0 || d1 == 0 || d2 == 0 || d3 == 0) return FTH_OK;
    FTH_ARG(src && dst, "permute: NULL operand");
    constexpr int EPV = 16 / sizeof(T);
    int vec = (d3 % EPV == 0 && ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) == 0) ? EPV : 1;
    int64_t total = d0 * d1 * d2 * (d3 / vec);
    int64_t grid = fth::ceil_div(total, kBlock);
    FTH_ARG(grid <= kMaxGrid, "permute: too long for one launch");
    permute_0213_kernel<T><<<dim3((unsigned)grid), dim3(kBlock), 0, fth::resolve_stream(s)>>>(src, dst, d0, d1, d2, d3, vec);
    FTH_CHECK_LAUNCH("permute_0213");
    return FTH_OK;
}

template <typename T>
int32_t launch_transpose(const T *src, T *dst, int64_t batch, int64_t rows, int64_t cols, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(batch >= 0 && rows >= 0 && cols >= 0, "transpose: negative extent");
    if (batch == 0 || rows == 0 || cols == 0) return FTH_OK;
    FTH_ARG(src && dst, "transpose: NULL operand");
    FTH_ARG(src != dst, "transpose: source and destination must not be the same buffer");
    constexpr int EPV = 16 / (int)sizeof(T);
    const bool vec = rows % EPV == 0 && cols % EPV == 0 &&
                     ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) == 0;
    const int ts = vec ? 64 : 32;
    const int64_t tiles_x = fth::ceil_div(cols, ts), tiles = tiles_x * fth::ceil_div(rows, ts);
    FTH_ARG(tiles <= kMaxGrid, "transpose: matrix too large for one launch");
    hipStream_t st = fth::resolve_stream(s);
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {  // the grid's second extent is limited to 65535
        const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        const T *sp = src + b0 * rows * cols;
        T *dp = dst + b0 * rows * cols;
        if (vec) transpose_tile_kernel<T><<<dim3((unsigned)tiles, (unsigned)nb), dim3(kBlock), 0, st>>>(sp, dp, rows, cols, tiles_x);
        else transpose_scalar_kernel<T><<<dim3((unsigned)tiles, (unsigned)nb), dim3(kBlock), 0, st>>>(sp, dp, rows, cols, tiles_x);
        FTH_CHECK_LAUNCH("transpose");
    }
    return FTH_OK;
}

}  // namespace

namespace fth {
int32_t argmax_from_group_max(const float *logits, int64_t rows, int64_t cols, const float *rowmax, int64_t groups, float *out,
                              hipStream_t st) {
    FTH_REQUIRE_DEVICE();
    if (rows <= 0) return FTH_OK;
    FTH_ARG(logits && rowmax && out && cols > 0 && groups == fth::gemm_rowmax_groups(cols),
            "argmax_from_group_max: the groups do not cover the columns");
    FTH_ARG(fth::ceil_div(rows, kGroupRows) <= kMaxGrid && groups <= 2147483647LL, "argmax_from_group_max: too many rows for one launch");
    argmax_group_kernel<<<dim3((unsigned)fth::ceil_div(rows, kGroupRows)), dim3(kGroupRows * kGroupSlices), 0, st>>>(logits, rows, cols, rowmax,
                                                                                                                   (int)groups, out);
    FTH_CHECK_LAUNCH("argmax_from_group_max");
    return FTH_OK;
}
}  // namespace fth

extern "C" {

int32_t fth_dev_index_select_f32(const float *input, int64_t outer, int64_t dim_size, int64_t inner,
                                 const double *indices, int64_t num_indices, float *out, int64_t *bad_index,
                                 fth_stream s) {
    return launch_index_select<float>(input, outer, dim_size, inner, indices, num_indices, out, bad_index, s);
}
int32_t fth_dev_index_select_f64(const double *input, int64_t outer, int64_t dim_size, int64_t inner,
                                 const double *indices, int64_t num_indices, double *out, int64_t *bad_index,
                                 fth_stream s) {
    return launch_index_select<double>(input, outer, dim_size, inner, indices, num_indices, out, bad_index, s);
}

int32_t fth_dev_embedding_add_f32(const float *wte, int64_t vocab, const float *wpe, int64_t max_pos,
                                  const double *ids, int64_t tokens, int64_t seq, int64_t width, float *out,
                                  int64_t *bad_index, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(vocab >= 0 && max_pos >= 0 && tokens >= 0 && seq >= 0 && width >= 0, "embedding: negative extent");
    hipStream_t st = fth::resolve_stream(s);
    if (bad_index) {
        set_i64_kernel<<<1, 1, 0, st>>>(bad_index, -1);
        FTH_CHECK_LAUNCH("embedding(bad_index reset)");
    }
    if (tokens == 0 || width == 0) return FTH_OK;
    FTH_ARG(seq > 0 && seq <= max_pos, "embedding: seq %lld exceeds the %lld learned positions", (long long)seq,
            (long long)max_pos);
    FTH_ARG(wte && wpe && ids && out, "embedding: NULL operand");
    int64_t grid = fth::ceil_div(tokens, kBlock / kWave);
    FTH_ARG(grid <= kMaxGrid, "embedding: too many tokens for one launch");
    embedding_add_kernel<<<dim3((unsigned)grid), dim3(kBlock), 0, st>>>(wte, vocab, wpe, ids, tokens, seq, width, out,
                                                                        bad_index);
    FTH_CHECK_LAUNCH("embedding_add");
    return FTH_OK;
}

int32_t fth_dev_argmax_f32(const float *x, int64_t outer, int64_t reduce, int64_t inner, float *out, fth_stream s) {
    return launch_argmax<float>(x, outer, reduce, inner, out, s);
}
int32_t fth_dev_argmax_f64(const double *x, int64_t outer, int64_t reduce, int64_t inner, double *out, fth_stream s) {
    return launch_argmax<double>(x, outer, reduce, inner, out, s);
}
int32_t fth_dev_transpose_2d_f32(const float *src, float *dst, int64_t rows, int64_t cols, fth_stream s) {
    return launch_transpose<float>(src, dst, 1, rows, cols, s);
}
int32_t fth_dev_transpose_2d_f64(const double *src, double *dst, int64_t rows, int64_t cols, fth_stream s) {
    return launch_transpose<double>(src, dst, 1, rows, cols, s);
}
int32_t fth_dev_transpose_batched_f32(const float *src, float *dst, int64_t batch, int64_t rows, int64_t cols, fth_stream s) {
    return launch_transpose<float>(src, dst, batch, rows, cols, s);
}
int32_t fth_dev_transpose_batched_f64(const double *src, double *dst, int64_t batch, int64_t rows, int64_t cols, fth_stream s) {
    return launch_transpose<double>(src, dst, batch, rows, cols, s);
}
int32_t fth_dev_permute_0213_f32(const float *src, float *dst, int64_t d0, int64_t d1, int64_t d2, int64_t d3,
                                 fth_stream s) {
    return launch_permute<float>(src, dst, d0, d1, d2, d3, s);
}
int32_t fth_dev_permute_0213_f64(const double *src, double *dst, int64_t d0, int64_t d1, int64_t d2, int64_t d3,
                                 fth_stream s) {
    return launch_permute<double>(src, dst, d0, d1, d2, d3, s);
}

}  // extern "C"
