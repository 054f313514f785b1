// Memory-bound row kernels for gfx950: last-dim softmax, LayerNorm, add+LayerNorm, RMSNorm,
// erf-GELU, add, bias add, bias+residual add.
//
// Shape of every row kernel: the fewest 64-lane wavefronts (1, 2, 4, 8 or 16) that keep a lane at
// four 128-bit vectors or fewer own one row (rows beyond 16 Ki elements grow the per-lane count to
// 8 or 16 vectors), pull it from HBM once with non-temporal 128-bit loads into registers, reduce
// with a fixed xor-butterfly over the wavefront and a fixed left-to-right fold over the row's
// wavefronts (one barrier per reduction, through alternating LDS halves), and write the row back
// once with non-temporal 128-bit stores. Elementwise kernels and the bias kernels hold one vector
// per thread. No atomics anywhere: the reduction tree is a function of (row length, kernel variant)
// only, so repeated runs are bitwise identical. Rows whose base is not 16-byte aligned, whose
// length is not a multiple of the vector width, or which do not fit the register budget take a
// block-per-row streaming variant with the same fixed trees.
//
// Arithmetic follows crates/ft-kernel-cpu/src/lib.rs step for step (separate multiplies and adds;
// this file is compiled with -ffp-contract=off): softmax :39219-39229, LayerNorm :5886-5909,
// add+LayerNorm :5946-5970, RMSNorm :6466-6480, GELU :36966-36969, add :36870-36877,
// bias pass :17336-17351. Only the summation ORDER differs (tree instead of sequential /
// pairwise-128), which is what the 1e-5 tolerance of the parity tests covers.

#include <algorithm>
#include <cstdlib>
#include <initializer_list>

#include "common.hpp"
#include "devmath.hpp"

namespace {

constexpr int kWave = 64;
constexpr int kBlock = 256;

// Streamed rows carry the non-temporal hint in both directions: a row is read once and written
// once, so it should not displace the reusable gamma / beta / bias lines. Measured on MI355X at
// fp32 [8192,4096] with every launch on a different buffer set (so that nothing is served from the
// 256 MB last-level cache): non-temporal loads gain 2-8 %, non-temporal stores 2-25 %. (Relaunching
// on ONE buffer set shows the opposite for loads, because the temporal loads then hit lines their
// own previous launch left in that cache.)
typedef float nat_f4 __attribute__((ext_vector_type(4)));
typedef double nat_d2 __attribute__((ext_vector_type(2)));
#ifndef FTH_NT_LOAD
#define FTH_NT_LOAD 1
#endif
#ifndef FTH_NT_STORE
#define FTH_NT_STORE 1
#endif
__device__ __forceinline__ float4 stream_load(const float4 *p) {
#if FTH_NT_LOAD
    nat_f4 v = __builtin_nontemporal_load(reinterpret_cast<const nat_f4 *>(p));
    return make_float4(v.x, v.y, v.z, v.w);
#else
    return *p;
#endif
}
__device__ __forceinline__ double2 stream_load(const double2 *p) {
#if FTH_NT_LOAD
    nat_d2 v = __builtin_nontemporal_load(reinterpret_cast<const nat_d2 *>(p));
    return make_double2(v.x, v.y);
#else
    return *p;
#endif
}
__device__ __forceinline__ void stream_store(float4 *p, const float4 &v) {
#if FTH_NT_STORE
    nat_f4 n = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(n, reinterpret_cast<nat_f4 *>(p));
#else
    *p = v;
#endif
}
__device__ __forceinline__ void stream_store(double2 *p, const double2 &v) {
#if FTH_NT_STORE
    nat_d2 n = {v.x, v.y};
    __builtin_nontemporal_store(n, reinterpret_cast<nat_d2 *>(p));
#else
    *p = v;
#endif
}

template <typename T> struct Vec128;
template <> struct Vec128<float> { using type = float4; static constexpr int n = 4; };
template <> struct Vec128<double> { using type = double2; static constexpr int n = 2; };

__device__ __forceinline__ float dev_exp(float x) { return fth::exp_hw(x); }
__device__ __forceinline__ double dev_exp(double x) { return exp(x); }
__device__ __forceinline__ float dev_sqrt(float x) { return sqrtf(x); }
__device__ __forceinline__ double dev_sqrt(double x) { return sqrt(x); }
__device__ __forceinline__ float dev_max(float a, float b) { return fmaxf(a, b); }
__device__ __forceinline__ double dev_max(double a, double b) { return fmax(a, b); }
__device__ __forceinline__ float dev_gelu(float x) { return fth::gelu_erf(x); }
__device__ __forceinline__ double dev_gelu(double x) {
    return (0.5 * x) * (1.0 + erf(x * 0.70710678118654752440));
}
// tanh-form GELU, 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))): the `gelu` kernel of the reference's fused GPU module
// (crates/ft-kernel-metal/src/fused.rs:301-313, with its |x| >= 10 clamp) and GELU::tanh() (crates/ft-nn/src/lib.rs:1924-1957).
__device__ __forceinline__ float dev_gelu_tanh(float x) {
    if (x >= 10.0f) return x;
    if (x <= -10.0f) return 0.0f;
    return 0.5f * x * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
}
__device__ __forceinline__ double dev_gelu_tanh(double x) {
    return 0.5 * x * (1.0 + tanh(0.79788456080286535588 * (x + 0.044715 * x * x * x)));
}
template <typename T> __device__ __forceinline__ T neg_inf();
template <> __device__ __forceinline__ float neg_inf<float>() { return -__builtin_inff(); }
template <> __device__ __forceinline__ double neg_inf<double>() { return -__builtin_inf(); }

struct SumOp {
    template <typename T> __device__ __forceinline__ T operator()(T a, T b) const { return a + b; }
};
struct MaxOp {
    template <typename T> __device__ __forceinline__ T operator()(T a, T b) const { return dev_max(a, b); }
};

// Fixed xor-butterfly over the 64 lanes; every lane ends with the same bits.
template <typename T, class F> __device__ __forceinline__ T wave_reduce(T v, F f) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = f(v, __shfl_xor(v, off, kWave));
    return v;
}

// Threads of the block that runs rows shared by WPR wavefronts: 256 (4 / WPR rows per block) up to
// WPR = 4, one row per block of 64 * WPR threads beyond.
template <int WPR> struct RowBlock {
    static constexpr int kThreads = WPR <= 4 ? kBlock : kWave * WPR;
    static constexpr int kRows = kThreads / (kWave * WPR);
    // A compute unit holds 2048 threads (8 wavefronts per SIMD) at up to 64 vector registers per
    // lane, 1536 at up to 85, 1024 at up to 128 and 512 at up to 256. `sets` counts the row-sized register sets the
    // kernel keeps (row, prefetched row, gamma, beta, second operand); a set is 4 * vpl registers. The result is
    // the second argument of __launch_bounds__, which hipcc reads as wavefronts per SIMD (not blocks per
    // compute unit): the register budget the kernel is compiled for, whatever its block size.
    static constexpr int min_blocks(int vpl, int sets, int elem_bytes) {
        const int regs = 4 * vpl * sets + 40;
        // (1536 threads: fp32 only; the fp64 kernels need the room for their exponential)
        const int threads = regs <= 64 ? 2048 : (regs <= 80 && elem_bytes == 4) ? 1536 : regs <= 128 ? 1024 : 512;
        const int waves = threads / 256, own = kThreads / 256;
        return waves > own ? waves : own;
    }
};
constexpr int kMaxWaves = 16;
// Rows of up to this many vectors per lane keep gamma / beta in registers; longer ones fetch them
// from cache at use.
constexpr int kHoistVpl = 2;

// Reduction over the WPR wavefronts that share a row (WPR == 1: the wavefront alone; otherwise the
// row's wavefronts inside the block, folded left to right through LDS). `smem` holds 2 * kMaxWaves
// values and consecutive calls alternate between its halves (`phase`), so one barrier per call is
// enough: a wavefront can only reach the write of call n + 2 after the barrier of call n + 1, which
// every wavefront reaches only after its reads of call n. Every thread of the block reaches the
// barriers (blocks with WPR > 1 never exit early).
template <int WPR, typename T, class F>
__device__ __forceinline__ T group_reduce(T v, F f, T *smem, int &phase) {
    v = wave_reduce(v, f);
    if constexpr (WPR == 1) {
        return v;
    } else {
        const int wave = threadIdx.x / kWave;
        const int first = (wave / WPR) * WPR;
        T *buf = smem + phase * kMaxWaves;
        phase ^= 1;
        if ((threadIdx.x & (kWave - 1)) == 0) buf[wave] = v;
        __syncthreads();
        T r = buf[first];
#pragma unroll
        for (int w = 1; w < WPR; ++w) r = f(r, buf[first + w]);
        return r;
    }
}

// ---------------------------------------------------------------------------------------------
// Register-resident row: VPL 128-bit vectors per lane, WPR wavefronts per row.
// ---------------------------------------------------------------------------------------------
template <typename T, int VPL, int WPR> struct RowRegs {
    using V = typename Vec128<T>::type;
    static constexpr int EPV = Vec128<T>::n;
    static constexpr int kLanes = WPR * kWave;
    T e[VPL][EPV];

    __device__ __forceinline__ static int lane() {
        return threadIdx.x & (kLanes - 1);
    }
    __device__ __forceinline__ void load(const T *row, int nvec, T fill) {
        const V *p = reinterpret_cast<const V *>(row);
        V tmp[VPL];
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            int v = lane() + i * kLanes;
            if (v < nvec) tmp[i] = stream_load(p + v);
        }
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            int v = lane() + i * kLanes;
            if (v < nvec) {
                unpack(tmp[i], e[i]);
            } else {
#pragma unroll
                for (int j = 0; j < EPV; ++j) e[i][j] = fill;
            }
        }
    }
    // Same lane layout, ordinary (cacheable) loads: for the per-column vectors every row re-reads.
    __device__ __forceinline__ void load_cached(const T *vec, int nvec, T fill) {
        const V *p = reinterpret_cast<const V *>(vec);
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            int v = lane() + i * kLanes;
            if (v < nvec) {
                unpack(p[v], e[i]);
            } else {
#pragma unroll
                for (int j = 0; j < EPV; ++j) e[i][j] = fill;
            }
        }
    }
    __device__ __forceinline__ static void unpack(const float4 &v, float *o) {
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    }
    __device__ __forceinline__ static void unpack(const double2 &v, double *o) {
        o[0] = v.x; o[1] = v.y;
    }
    __device__ __forceinline__ static float4 pack(const float *o) { return make_float4(o[0], o[1], o[2], o[3]); }
    __device__ __forceinline__ static double2 pack(const double *o) { return make_double2(o[0], o[1]); }
    __device__ __forceinline__ static void load_vec(const T *base, int v, T *o) {
        unpack(reinterpret_cast<const V *>(base)[v], o);
    }
    __device__ __forceinline__ void store(T *row, int nvec) const {
        V *p = reinterpret_cast<V *>(row);
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            int v = lane() + i * kLanes;
            if (v < nvec) stream_store(p + v, pack(e[i]));
        }
    }
};

// The rows of one row group (the WPR wavefronts that share a row). Group g of G takes rows g, g + G,
// g + 2 G, ... for `iters` turns, the same count in every group so that all wavefronts of a block
// meet at the same barriers; a turn past the last row works on a clamped copy of it and stores
// nothing. Neighbouring groups are on neighbouring rows at any time, and a group keeps its
// per-column vectors (gamma, beta) in registers across its rows: with one row per block those
// vectors, 32 KiB per fp32 row of 4096, crossed the L2 -> L1 path once per row, twice the volume
// of the row itself, and LayerNorm ran at 0.63 of the HBM peak against 0.77 without them.
template <int WPR> struct RowWalk {
    int64_t row, stride, last;
    __device__ __forceinline__ RowWalk(int64_t rows)
        : row((int64_t)blockIdx.x * RowBlock<WPR>::kRows + threadIdx.x / (kWave * WPR)),
          stride((int64_t)gridDim.x * RowBlock<WPR>::kRows), last(rows - 1) {}
    __device__ __forceinline__ int64_t clamped(int64_t r) const { return r < last ? r : last; }
    __device__ __forceinline__ bool live() const { return row <= last; }
};
// The next row is requested before the current one is reduced when a second register set fits.
template <int VPL> constexpr bool kPrefetch = VPL <= 4;

// ---- softmax ------------------------------------------------------------------------------
template <typename T, int VPL, int WPR>
__global__ __launch_bounds__(RowBlock<WPR>::kThreads, RowBlock<WPR>::min_blocks(VPL, 2, (int)sizeof(T))) void softmax_row_kernel(
    const T *__restrict__ x, T *__restrict__ y, int64_t rows, int cols, int iters) {
    __shared__ T smem[2 * kMaxWaves];
    int phase = 0;
    using R = RowRegs<T, VPL, WPR>;
    const int nvec = cols / R::EPV;
    RowWalk<WPR> walk(rows);
    R r, nxt;
    r.load(x + walk.clamped(walk.row) * cols, nvec, neg_inf<T>());
    for (int it = 0; it < iters; ++it) {
        if constexpr (kPrefetch<VPL>) {
            if (it + 1 < iters) nxt.load(x + walk.clamped(walk.row + walk.stride) * cols, nvec, neg_inf<T>());
        }
        T m = neg_inf<T>();
#pragma unroll
        for (int i = 0; i < VPL; ++i)
#pragma unroll
            for (int j = 0; j < R::EPV; ++j) m = dev_max(m, r.e[i][j]);
        m = group_reduce<WPR>(m, MaxOp{}, smem, phase);
        T s = 0;
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            const bool live = (R::lane() + i * R::kLanes) < nvec;
#pragma unroll
            for (int j = 0; j < R::EPV; ++j) {
                // Padding slots must stay out of the sum even when m is -inf or NaN.
                T ev = live ? dev_exp(r.e[i][j] - m) : T(0);
                r.e[i][j] = ev;
                s += ev;
            }
        }
        s = group_reduce<WPR>(s, SumOp{}, smem, phase);
        // One correctly rounded 1 / s per row, then a multiply per element (the reference divides each
        // element: the two differ by at most one rounding, far inside the parity tolerance, and the
        // per-element IEEE division sequence would make this kernel ALU-bound).
        const T inv = T(1) / s;
#pragma unroll
        for (int i = 0; i < VPL; ++i)
#pragma unroll
            for (int j = 0; j < R::EPV; ++j) r.e[i][j] = r.e[i][j] * inv;
        r.store(y + walk.clamped(walk.row) * cols, walk.live() ? nvec : 0);
        walk.row += walk.stride;
        if (it + 1 < iters) {
            if constexpr (kPrefetch<VPL>) r = nxt;
            else r.load(x + walk.clamped(walk.row) * cols, nvec, neg_inf<T>());
        }
    }
}

// ---- LayerNorm / add+LayerNorm ---------------------------------------------------------------
template <typename T, int VPL, int WPR, bool ADD>
__global__ __launch_bounds__(RowBlock<WPR>::kThreads, RowBlock<WPR>::min_blocks(VPL, ADD ? 5 : 4, (int)sizeof(T))) void layernorm_row_kernel(
    const T *__restrict__ x, const T *__restrict__ x2, const T *__restrict__ w, const T *__restrict__ b, T *__restrict__ y,
    int64_t rows, int cols, T eps, int iters) {
    __shared__ T smem[2 * kMaxWaves];
    int phase = 0;
    using R = RowRegs<T, VPL, WPR>;
    const int nvec = cols / R::EPV;
    RowWalk<WPR> walk(rows);
    const T inv_n = T(1) / (T)cols;
    R rw, rb;  // gamma / beta of this lane's columns, kept for every row of the group
    if constexpr (VPL <= kHoistVpl) {
        if (w) rw.load_cached(w, nvec, T(1));
        if (b) rb.load_cached(b, nvec, T(0));
    }
    R r, nxt, nxt2;
    if constexpr (kPrefetch<VPL>) {
        r.load(x + walk.clamped(walk.row) * cols, nvec, T(0));
        if constexpr (ADD) nxt2.load(x2 + walk.clamped(walk.row) * cols, nvec, T(0));
    }
    for (int it = 0; it < iters; ++it) {
        if constexpr (!kPrefetch<VPL>) {
            r.load(x + walk.clamped(walk.row) * cols, nvec, T(0));
            if constexpr (ADD) nxt2.load(x2 + walk.clamped(walk.row) * cols, nvec, T(0));
        }
        if constexpr (ADD) {
#pragma unroll
            for (int i = 0; i < VPL; ++i)
#pragma unroll
                for (int j = 0; j < R::EPV; ++j) r.e[i][j] = r.e[i][j] + nxt2.e[i][j];
        }
        if constexpr (kPrefetch<VPL>) {
            if (it + 1 < iters) {
                nxt.load(x + walk.clamped(walk.row + walk.stride) * cols, nvec, T(0));
                if constexpr (ADD) nxt2.load(x2 + walk.clamped(walk.row + walk.stride) * cols, nvec, T(0));
            }
        }
        T sum = 0;
#pragma unroll
        for (int i = 0; i < VPL; ++i)
#pragma unroll
            for (int j = 0; j < R::EPV; ++j) sum += r.e[i][j];
        sum = group_reduce<WPR>(sum, SumOp{}, smem, phase);
        const T mean = sum * inv_n;
        T vsum = 0;
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            const bool live = (R::lane() + i * R::kLanes) < nvec;
#pragma unroll
            for (int j = 0; j < R::EPV; ++j) {
                T d = r.e[i][j] - mean;
                vsum += live ? d * d : T(0);
            }
        }
        vsum = group_reduce<WPR>(vsum, SumOp{}, smem, phase);
        const T rstd = T(1) / dev_sqrt(vsum * inv_n + eps);
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            const int v = R::lane() + i * R::kLanes;
            if (v < nvec) {
                T wv[R::EPV], bv[R::EPV];
                if constexpr (VPL > kHoistVpl) {
                    if (w) R::load_vec(w, v, wv);
                    if (b) R::load_vec(b, v, bv);
                }
#pragma unroll
                for (int j = 0; j < R::EPV; ++j) {
                    T o = (r.e[i][j] - mean) * rstd;
                    if (w) o = o * (VPL <= kHoistVpl ? rw.e[i][j] : wv[j]);
                    if (b) o = o + (VPL <= kHoistVpl ? rb.e[i][j] : bv[j]);
                    r.e[i][j] = o;
                }
            }
        }
        r.store(y + walk.clamped(walk.row) * cols, walk.live() ? nvec : 0);
        walk.row += walk.stride;
        if constexpr (kPrefetch<VPL>) {
            if (it + 1 < iters) r = nxt;
        }
    }
}

// ---- LayerNorm, RPT rows side by side per row group ---------------------------------------------
// A lane holds the same columns of RPT consecutive rows, so gamma and beta are fetched once per RPT rows (with one row
// per block they crossed the L2 -> L1 path once per row, 32 KiB for every 16 KiB fp32 row of 4096) and the RPT
// reductions share their barriers. Per row the arithmetic and the reduction tree are those of layernorm_row_kernel:
// the two kernels give the same bits.
template <int WPR, int N, typename T>
__device__ __forceinline__ void group_sum_n(T (&v)[N], T *smem, int &phase) {
#pragma unroll
    for (int j = 0; j < N; ++j) v[j] = wave_reduce(v[j], SumOp{});
    if constexpr (WPR > 1) {
        const int wave = threadIdx.x / kWave;
        const int first = (wave / WPR) * WPR;
        T *buf = smem + phase * (kMaxWaves * N);
        phase ^= 1;
        if ((threadIdx.x & (kWave - 1)) == 0) {
#pragma unroll
            for (int j = 0; j < N; ++j) buf[wave * N + j] = v[j];
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < N; ++j) {
            T r = buf[first * N + j];
#pragma unroll
            for (int w = 1; w < WPR; ++w) r = r + buf[(first + w) * N + j];
            v[j] = r;
        }
    }
}

template <typename T, int VPL, int WPR, int RPT>
__global__ __launch_bounds__(RowBlock<WPR>::kThreads) void layernorm_rows_kernel(const T *__restrict__ x, const T *__restrict__ w,
                                                                                 const T *__restrict__ b, T *__restrict__ y,
                                                                                 int64_t rows, int cols, T eps) {
    __shared__ T smem[2 * kMaxWaves * RPT];
    int phase = 0;
    using R = RowRegs<T, VPL, WPR>;
    const int nvec = cols / R::EPV;
    const T inv_n = T(1) / (T)cols;
    const int64_t row0 = ((int64_t)blockIdx.x * RowBlock<WPR>::kRows + threadIdx.x / (kWave * WPR)) * RPT;
    R r[RPT];
#pragma unroll
    for (int q = 0; q < RPT; ++q) {
        const int64_t row = row0 + q < rows ? row0 + q : rows - 1;  // a turn past the last row works on a copy of it and stores nothing
        r[q].load(x + row * cols, nvec, T(0));
    }
    T sum[RPT];
#pragma unroll
    for (int q = 0; q < RPT; ++q) {
        sum[q] = 0;
#pragma unroll
        for (int i = 0; i < VPL; ++i)
#pragma unroll
            for (int j = 0; j < R::EPV; ++j) sum[q] += r[q].e[i][j];
    }
    group_sum_n<WPR, RPT>(sum, smem, phase);
    T mean[RPT], vsum[RPT];
#pragma unroll
    for (int q = 0; q < RPT; ++q) {
        mean[q] = sum[q] * inv_n;
        vsum[q] = 0;
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            const bool live = (R::lane() + i * R::kLanes) < nvec;
#pragma unroll
            for (int j = 0; j < R::EPV; ++j) {
                const T d = r[q].e[i][j] - mean[q];
                vsum[q] += live ? d * d : T(0);
            }
        }
    }
    group_sum_n<WPR, RPT>(vsum, smem, phase);
    T rstd[RPT];
#pragma unroll
    for (int q = 0; q < RPT; ++q) rstd[q] = T(1) / dev_sqrt(vsum[q] * inv_n + eps);
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
        const int v = R::lane() + i * R::kLanes;
        if (v < nvec) {
            T wv[R::EPV], bv[R::EPV];
            if (w) R::load_vec(w, v, wv);
            if (b) R::load_vec(b, v, bv);
#pragma unroll
            for (int q = 0; q < RPT; ++q)
#pragma unroll
                for (int j = 0; j < R::EPV; ++j) {
                    T o = (r[q].e[i][j] - mean[q]) * rstd[q];
                    if (w) o = o * wv[j];
                    if (b) o = o + bv[j];
                    r[q].e[i][j] = o;
                }
        }
    }
#pragma unroll
    for (int q = 0; q < RPT; ++q) r[q].store(y + (row0 + q < rows ? row0 + q : rows - 1) * cols, row0 + q < rows ? nvec : 0);
}

// Direct global -> LDS copy of 16 bytes per lane: the wavefront's 64 lanes fill 1 KiB of LDS at `lds_byte` in lane
// order, with no staging registers. The compiler does not see the LDS write, so the reader waits for vmcnt(0) itself.
__device__ __forceinline__ void vec_to_lds(const void *base, unsigned lane_bytes, unsigned lds_byte) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_bytes), "s"(base),
                 "s"(__builtin_amdgcn_readfirstlane(lds_byte))
                 : "memory", "m0");
}
template <typename T> __device__ __forceinline__ const T *uniform_base(const T *ptr) {
    const uint64_t v = reinterpret_cast<uint64_t>(ptr);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<const T *>(((uint64_t)hi << 32) | lo);
}

// ---- RMSNorm ---------------------------------------------------------------------------------
template <typename T, int VPL, int WPR>
__global__ __launch_bounds__(RowBlock<WPR>::kThreads, RowBlock<WPR>::min_blocks(VPL, 3, (int)sizeof(T))) void rmsnorm_row_kernel(
    const T *__restrict__ x, const T *__restrict__ w, T *__restrict__ y, int64_t rows, int cols, T eps, int iters) {
    __shared__ T smem[2 * kMaxWaves];
    int phase = 0;
    using R = RowRegs<T, VPL, WPR>;
    const int nvec = cols / R::EPV;
    RowWalk<WPR> walk(rows);
    const T inv_n = T(1) / (T)cols;
    R rw;
    if constexpr (VPL <= kHoistVpl) {
        if (w) rw.load_cached(w, nvec, T(1));
    }
    R r, nxt;
    r.load(x + walk.clamped(walk.row) * cols, nvec, T(0));
    for (int it = 0; it < iters; ++it) {
        if constexpr (kPrefetch<VPL>) {
            if (it + 1 < iters) nxt.load(x + walk.clamped(walk.row + walk.stride) * cols, nvec, T(0));
        }
        T ss = 0;
#pragma unroll
        for (int i = 0; i < VPL; ++i)
#pragma unroll
            for (int j = 0; j < R::EPV; ++j) ss += r.e[i][j] * r.e[i][j];
        ss = group_reduce<WPR>(ss, SumOp{}, smem, phase);
        const T rstd = T(1) / dev_sqrt(ss * inv_n + eps);
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            const int v = R::lane() + i * R::kLanes;
            if (v < nvec) {
                T wv[R::EPV];
                if constexpr (VPL > kHoistVpl) {
                    if (w) R::load_vec(w, v, wv);
                }
#pragma unroll
                for (int j = 0; j < R::EPV; ++j) {
                    T o = r.e[i][j] * rstd;
                    if (w) o = o * (VPL <= kHoistVpl ? rw.e[i][j] : wv[j]);
                    r.e[i][j] = o;
                }
            }
        }
        r.store(y + walk.clamped(walk.row) * cols, walk.live() ? nvec : 0);
        walk.row += walk.stride;
        if (it + 1 < iters) {
            if constexpr (kPrefetch<VPL>) r = nxt;
            else r.load(x + walk.clamped(walk.row) * cols, nvec, T(0));
        }
    }
}

// ---- Row ops, walking rows: few workgroups, each owning rows r, r + G, r + 2 G, ... ---------------
// Two 512-lane workgroups per compute unit, each in a plain load -> reduce -> store loop over its rows, with the
// per-column vectors (gamma, beta) copied into LDS once per workgroup. Same arithmetic and reduction trees as the
// one-row-per-workgroup kernels above (the results are bit-identical); what changes is how the memory system is driven.
enum class RowOp { Softmax, LayerNorm, RmsNorm };

template <typename T, int VPL, int WPR, RowOp OP>
__global__ __launch_bounds__(RowBlock<WPR>::kThreads) void row_walk_kernel(const T *__restrict__ x, const T *__restrict__ w,
                                                                           const T *__restrict__ b, T *__restrict__ y,
                                                                           int64_t rows, int cols, T eps) {
    static_assert(RowBlock<WPR>::kRows == 1, "one row group per workgroup");
    constexpr int NT = RowBlock<WPR>::kThreads;
    using R = RowRegs<T, VPL, WPR>;
    using V = typename Vec128<T>::type;
    extern __shared__ __align__(16) unsigned char dyn_lds[];  // the only LDS object (offset 0): gamma, beta, exchange buffer
    T *smem = reinterpret_cast<T *>(dyn_lds + (size_t)2 * VPL * NT * 16);
    int phase = 0;
    const int nvec = cols / R::EPV;
    const T inv_n = T(1) / (T)cols;
    const bool has_w = OP != RowOp::Softmax && w != nullptr, has_b = OP == RowOp::LayerNorm && b != nullptr;
    if constexpr (OP != RowOp::Softmax) {
        const unsigned wave_byte = (threadIdx.x / kWave) * (kWave * 16);
#pragma unroll
        for (int i = 0; i < VPL; ++i) {
            int v = (int)threadIdx.x + i * NT;
            v = v < nvec ? v : nvec - 1;
            if (has_w) vec_to_lds(uniform_base(w), (unsigned)v * 16u, (unsigned)(i * NT * 16) + wave_byte);
            if (has_b) vec_to_lds(uniform_base(b), (unsigned)v * 16u, (unsigned)((VPL + i) * NT * 16) + wave_byte);
        }
    }
    const V *lw = reinterpret_cast<const V *>(dyn_lds), *lb = lw + VPL * NT;
    bool first = OP != RowOp::Softmax;
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
        R r;
        r.load(x + row * cols, nvec, OP == RowOp::Softmax ? neg_inf<T>() : T(0));
        if (first) {
            // gamma / beta were requested before the first row and vector memory operations complete in issue order;
            // the explicit wait is for the compiler, which does not know of the LDS writes.
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            first = false;
        }
        if constexpr (OP == RowOp::Softmax) {
            T m = neg_inf<T>();
#pragma unroll
            for (int i = 0; i < VPL; ++i)
#pragma unroll
                for (int j = 0; j < R::EPV; ++j) m = dev_max(m, r.e[i][j]);
            m = group_reduce<WPR>(m, MaxOp{}, smem, phase);
            T s = 0;
#pragma unroll
            for (int i = 0; i < VPL; ++i) {
                const bool live = (R::lane() + i * R::kLanes) < nvec;
#pragma unroll
                for (int j = 0; j < R::EPV; ++j) {
                    T ev = live ? dev_exp(r.e[i][j] - m) : T(0);
                    r.e[i][j] = ev;
                    s += ev;
                }
            }
            s = group_reduce<WPR>(s, SumOp{}, smem, phase);
            const T inv = T(1) / s;
#pragma unroll
            for (int i = 0; i < VPL; ++i)
#pragma unroll
                for (int j = 0; j < R::EPV; ++j) r.e[i][j] = r.e[i][j] * inv;
        } else {
            T mean = 0, rstd;
            if constexpr (OP == RowOp::LayerNorm) {
                T sum = 0;
#pragma unroll
                for (int i = 0; i < VPL; ++i)
#pragma unroll
                    for (int j = 0; j < R::EPV; ++j) sum += r.e[i][j];
                sum = group_reduce<WPR>(sum, SumOp{}, smem, phase);
                mean = sum * inv_n;
                T vsum = 0;
#pragma unroll
                for (int i = 0; i < VPL; ++i) {
                    const bool live = (R::lane() + i * R::kLanes) < nvec;
#pragma unroll
                    for (int j = 0; j < R::EPV; ++j) {
                        const T d = r.e[i][j] - mean;
                        vsum += live ? d * d : T(0);
                    }
                }
                vsum = group_reduce<WPR>(vsum, SumOp{}, smem, phase);
                rstd = T(1) / dev_sqrt(vsum * inv_n + eps);
            } else {
                T ss = 0;
#pragma unroll
                for (int i = 0; i < VPL; ++i)
#pragma unroll
                    for (int j = 0; j < R::EPV; ++j) ss += r.e[i][j] * r.e[i][j];
                ss = group_reduce<WPR>(ss, SumOp{}, smem, phase);
                rstd = T(1) / dev_sqrt(ss * inv_n + eps);
            }
#pragma unroll
            for (int i = 0; i < VPL; ++i) {
                const int v = R::lane() + i * R::kLanes;
                if (v < nvec) {
                    T wv[R::EPV], bv[R::EPV];
                    if (has_w) R::unpack(lw[i * NT + threadIdx.x], wv);
                    if (has_b) R::unpack(lb[i * NT + threadIdx.x], bv);
#pragma unroll
                    for (int j = 0; j < R::EPV; ++j) {
                        T o = OP == RowOp::LayerNorm ? (r.e[i][j] - mean) * rstd : r.e[i][j] * rstd;
                        if (has_w) o = o * wv[j];
                        if (has_b) o = o + bv[j];
                        r.e[i][j] = o;
                    }
                }
            }
        }
        r.store(y + row * cols, nvec);
    }
}

// Launches row_walk_kernel when the shape fits it (rows of 513 to 1024 vectors, enough rows to give every workgroup a
// few); returns false when the caller should take its one-row-per-workgroup path.
template <typename T, RowOp OP>
bool try_row_walk(const T *x, const T *w, const T *b, T *y, int64_t rows, int64_t cols, T eps, int vpl, int wpr, hipStream_t st) {
    // Measured at fp32 [8192, 4096] on rotating buffers, fractions of the HBM peak, one row per workgroup against walking
    // with 2 / 3 / 4 workgroups per compute unit: LayerNorm (gamma and beta) 0.724 against 0.751 / 0.713 / 0.711; RMSNorm
    // 0.760 against 0.759 / 0.739 / 0.743; softmax 0.775 against 0.750 / 0.715 / 0.723. So only the op that reads two
    // per-column vectors walks by default.
    static const int forced = [] {
        const char *e = std::getenv("FT_HIP_ROW_WALK");  // tuning knob: workgroups per compute unit of the walking kernel, every op (0 = off)
        return e ? std::atoi(e) : -1;
    }();
    const int per_cu = forced >= 0 ? forced : (OP == RowOp::LayerNorm && w != nullptr && b != nullptr) ? 2 : 0;
    if (per_cu <= 0 || wpr != 8 || vpl != 2) return false;
    const int cus = fth::compute_units() > 0 ? fth::compute_units() : 256;
    const int64_t grid = (int64_t)cus * per_cu;
    if (rows < 4 * grid) return false;
    const size_t lds = (size_t)2 * 2 * 512 * 16 + 2 * kMaxWaves * sizeof(T);
    row_walk_kernel<T, 2, 8, OP><<<dim3((unsigned)grid), dim3(512), lds, st>>>(x, w, b, y, rows, (int)cols, eps);
    return true;
}

// ---------------------------------------------------------------------------------------------
// Streaming variants: one 256-thread block per row, scalar loads, the row is re-read from L2.
// ---------------------------------------------------------------------------------------------
template <typename T, class F>
__device__ __forceinline__ T block_reduce(T v, F f, T *smem, int &phase) {
    return group_reduce<4>(v, f, smem, phase);
}

template <typename T>
__global__ __launch_bounds__(kBlock) void softmax_stream_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                                int64_t rows, int64_t cols) {
    __shared__ T smem[2 * kMaxWaves];
    int phase = 0;
    const T *xr = x + (int64_t)blockIdx.x * cols;
    T *yr = y + (int64_t)blockIdx.x * cols;
    T m = neg_inf<T>();
    for (int64_t j = threadIdx.x; j < cols; j += kBlock) m = dev_max(m, xr[j]);
    m = block_reduce(m, MaxOp{}, smem, phase);
    T s = 0;
    for (int64_t j = threadIdx.x; j < cols; j += kBlock) {
        T ev = dev_exp(xr[j] - m);
        yr[j] = ev;
        s += ev;
    }
    s = block_reduce(s, SumOp{}, smem, phase);
    for (int64_t j = threadIdx.x; j < cols; j += kBlock) yr[j] = yr[j] / s;
}

// Softmax over the middle dim of [outer, reduce, inner]: one thread per (outer, inner) lane of
// the tensor, coalesced along inner, sequential over reduce (crates/ft-kernel-cpu/src/lib.rs:
// 39244-39260; the sum there is pairwise-128, here sequential: tolerance parity).
template <typename T>
__global__ __launch_bounds__(kBlock) void softmax_strided_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                                 int64_t outer, int64_t reduce, int64_t inner) {
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (idx >= outer * inner) return;
    const int64_t o = idx / inner, in = idx % inner;
    const T *xb = x + o * reduce * inner + in;
    T *yb = y + o * reduce * inner + in;
    T m = neg_inf<T>();
    for (int64_t r = 0; r < reduce; ++r) m = dev_max(m, xb[r * inner]);
    T s = 0;
    for (int64_t r = 0; r < reduce; ++r) {
        T ev = dev_exp(xb[r * inner] - m);
        yb[r * inner] = ev;
        s += ev;
    }
    for (int64_t r = 0; r < reduce; ++r) yb[r * inner] = yb[r * inner] / s;
}

template <typename T, bool ADD>
__global__ __launch_bounds__(kBlock) void layernorm_stream_kernel(const T *__restrict__ x, const T *__restrict__ x2,
                                                                  const T *__restrict__ w, const T *__restrict__ b,
                                                                  T *__restrict__ y, int64_t rows, int64_t cols,
                                                                  T eps) {
    __shared__ T smem[2 * kMaxWaves];
    int phase = 0;
    const T *xr = x + (int64_t)blockIdx.x * cols;
    const T *x2r = ADD ? x2 + (int64_t)blockIdx.x * cols : nullptr;
    T *yr = y + (int64_t)blockIdx.x * cols;
    const T inv_n = T(1) / (T)cols;
    T sum = 0;
    for (int64_t j = threadIdx.x; j < cols; j += kBlock) {
        T v = xr[j];
        if constexpr (ADD) {
            v = v + x2r[j];
            yr[j] = v;  // materialise a + b once, as the reference does
        }
        sum += v;
    }
    sum = block_reduce(sum, SumOp{}, smem, phase);
    const T mean = sum * inv_n;
    const T *src = ADD ? yr : xr;
    T vsum = 0;
    for (int64_t j = threadIdx.x; j < cols; j += kBlock) {
        T d = src[j] - mean;
        vsum += d * d;
    }
    vsum = block_reduce(vsum, SumOp{}, smem, phase);
    const T rstd = T(1) / dev_sqrt(vsum * inv_n + eps);
    for (int64_t j = threadIdx.x; j < cols; j += kBlock) {
        T o = (src[j] - mean) * rstd;
        if (w) o = o * w[j];
        if (b) o = o + b[j];
        yr[j] = o;
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void rmsnorm_stream_kernel(const T *__restrict__ x, const T *__restrict__ w,
                                                                T *__restrict__ y, int64_t rows, int64_t cols, T eps) {
    __shared__ T smem[2 * kMaxWaves];
    int phase = 0;
    const T *xr = x + (int64_t)blockIdx.x * cols;
    T *yr = y + (int64_t)blockIdx.x * cols;
    const T inv_n = T(1) / (T)cols;
    T ss = 0;
    for (int64_t j = threadIdx.x; j < cols; j += kBlock) ss += xr[j] * xr[j];
    ss = block_reduce(ss, SumOp{}, smem, phase);
    const T rstd = T(1) / dev_sqrt(ss * inv_n + eps);
    for (int64_t j = threadIdx.x; j < cols; j += kBlock) {
        T o = xr[j] * rstd;
        if (w) o = o * w[j];
        yr[j] = o;
    }
}

// ---------------------------------------------------------------------------------------------
// Elementwise: GELU, add. Each thread owns UNR 128-bit vectors a block-stride apart, loads them
// all before the first use, and a scalar tail covers what is left.
// ---------------------------------------------------------------------------------------------
enum class Ew { Gelu, Add, GeluTanh, Copy };

template <typename T, Ew OP, int UNR, int BT>
__global__ __launch_bounds__(BT) void elementwise_vec_kernel(const T *__restrict__ a, const T *__restrict__ b,
                                                             T *__restrict__ y, int64_t nvec) {
    using R = RowRegs<T, 1, 1>;
    using V = typename Vec128<T>::type;
    const int64_t base = (int64_t)blockIdx.x * (BT * UNR) + threadIdx.x;
    V va[UNR], vb[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
        int64_t v = base + (int64_t)u * BT;
        if (v < nvec) {
            va[u] = stream_load(reinterpret_cast<const V *>(a) + v);
            if constexpr (OP == Ew::Add) vb[u] = stream_load(reinterpret_cast<const V *>(b) + v);
        }
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
        int64_t v = base + (int64_t)u * BT;
        if (v < nvec) {
            T ea[R::EPV], eb[R::EPV];
            R::unpack(va[u], ea);
            if constexpr (OP == Ew::Add) R::unpack(vb[u], eb);
#pragma unroll
            for (int j = 0; j < R::EPV; ++j) {
                if constexpr (OP == Ew::Gelu) ea[j] = dev_gelu(ea[j]);
                else if constexpr (OP == Ew::GeluTanh) ea[j] = dev_gelu_tanh(ea[j]);
                else if constexpr (OP == Ew::Add) ea[j] = ea[j] + eb[j];
            }
            stream_store(reinterpret_cast<V *>(y) + v, R::pack(ea));
        }
    }
}

template <typename T, Ew OP>
__global__ __launch_bounds__(kBlock) void elementwise_scalar_kernel(const T *__restrict__ a, const T *__restrict__ b,
                                                                    T *__restrict__ y, int64_t begin, int64_t n) {
    const int64_t i = begin + (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    if constexpr (OP == Ew::Gelu) y[i] = dev_gelu(a[i]);
    else if constexpr (OP == Ew::GeluTanh) y[i] = dev_gelu_tanh(a[i]);
    else if constexpr (OP == Ew::Add) y[i] = a[i] + b[i];
    else y[i] = a[i];
}

// ---- bias add / bias + residual add: y[r, j] = (x[r, j] + bias[j]) (+ res[r, j]) --------------
// One 128-bit vector per thread over the flattened tensor; the bias vector is the vector index
// modulo the vectors of a row (the bias stays in cache).
template <typename T, bool RES, int BT>
__global__ __launch_bounds__(BT) void bias_flat_kernel(const T *x, const T *__restrict__ bias, const T *res, T *y,
                                                       int64_t total_vec, int row_vec) {
    using R = RowRegs<T, 1, 1>;
    using V = typename Vec128<T>::type;
    const int64_t v = (int64_t)blockIdx.x * BT + threadIdx.x;
    if (v >= total_vec) return;
    const int bv = (int)(v % row_vec);
    const V vx = stream_load(reinterpret_cast<const V *>(x) + v);
    const V vb = reinterpret_cast<const V *>(bias)[bv];
    V vr;
    if constexpr (RES) vr = stream_load(reinterpret_cast<const V *>(res) + v);
    T ex[R::EPV], eb[R::EPV], er[R::EPV];
    R::unpack(vx, ex);
    R::unpack(vb, eb);
    if constexpr (RES) R::unpack(vr, er);
#pragma unroll
    for (int j = 0; j < R::EPV; ++j) {
        T o = ex[j] + eb[j];
        if constexpr (RES) o = o + er[j];
        ex[j] = o;
    }
    stream_store(reinterpret_cast<V *>(y) + v, R::pack(ex));
}

template <typename T, bool RES>
__global__ __launch_bounds__(kBlock) void bias_scalar_kernel(const T *x, const T *__restrict__ bias,
                                                             const T *res, T *y, int64_t rows, int64_t cols) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= rows * cols) return;
    T o = x[i] + bias[i % cols];
    if constexpr (RES) o = o + res[i];
    y[i] = o;
}

// ---------------------------------------------------------------------------------------------
// Host-side dispatch
// ---------------------------------------------------------------------------------------------
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr int64_t kMaxGrid = 2147483647LL;

// Picks (VPL, WPR) for a register-resident row of `nvec` vectors, or returns false. Measured on
// MI355X over rotating buffers (rows x cols = 32 Mi fp32 elements): a row streams fastest from the
// fewest wavefronts that keep a lane at 4 vectors or fewer -- 768 and 1024 columns on one wavefront
// (0.75 of the HBM peak; 0.70 on two, 0.57 on four), 2048 on two, 4096 on four, 8192 and 16384 on
// eight with 4 and 8 vectors per lane. Sixteen wavefronts (one 1024-thread block per row) lose
// everywhere below 8192 columns. `max_vpl` caps the vectors a lane may hold.
inline bool pick_row_shape(int64_t nvec, int max_vpl, int &vpl, int &wpr) {
    if (nvec <= 0 || nvec > 64 * kMaxWaves * (int64_t)max_vpl) return false;
    static const int forced = [] {
        const char *e = std::getenv("FT_HIP_ROW_WPR");  // tuning knob: wavefronts per row (1, 2, 4, 8 or 16)
        return e ? std::atoi(e) : 0;
    }();
    // (rows of 769 to 1024 vectors on eight wavefronts, two vectors a lane: at fp32 [8192, 4096] on rotating buffers softmax
    // 0.754 -> 0.777 of the HBM peak, LayerNorm 0.719 -> 0.725, RMSNorm 0.739 -> 0.746 against four wavefronts with four vectors)
    int w = nvec <= 256 ? 1 : nvec <= 512 ? 2 : nvec <= 768 ? 4 : nvec <= 4096 ? 8 : 16;
    if (forced == 1 || forced == 2 || forced == 4 || forced == 8 || forced == 16) {
        if (fth::ceil_div(nvec, 64 * forced) <= max_vpl) w = forced;
    }
    const int64_t need = fth::ceil_div(nvec, 64 * w);
    if (w == 16 && need > 8) return false;  // 1024 threads leave a lane 128 registers: 8 vectors at most
    vpl = need <= 1 ? 1 : need <= 2 ? 2 : need <= 4 ? 4 : need <= 8 ? 8 : 16;
    wpr = w;
    return true;
}

#define FTH_ROW_DISPATCH_VPL(VPL_, W_, LAUNCH)           \
    switch (VPL_) {                                      \
        case 1: { LAUNCH(1, W_); } break;                \
        case 2: { LAUNCH(2, W_); } break;                \
        case 4: { LAUNCH(4, W_); } break;                \
        case 8: { LAUNCH(8, W_); } break;                \
        default: { LAUNCH(16, W_); } break;              \
    }
#define FTH_ROW_DISPATCH(VPL_, WPR_, LAUNCH)                         \
    do {                                                             \
        switch (WPR_) {                                              \
            case 1: FTH_ROW_DISPATCH_VPL(VPL_, 1, LAUNCH) break;     \
            case 2: FTH_ROW_DISPATCH_VPL(VPL_, 2, LAUNCH) break;     \
            case 4: FTH_ROW_DISPATCH_VPL(VPL_, 4, LAUNCH) break;     \
            case 8: FTH_ROW_DISPATCH_VPL(VPL_, 8, LAUNCH) break;     \
            default:                                                 \
                switch (VPL_) {                                      \
                    case 1: { LAUNCH(1, 16); } break;                \
                    case 2: { LAUNCH(2, 16); } break;                \
                    case 4: { LAUNCH(4, 16); } break;                \
                    default: { LAUNCH(8, 16); } break;               \
                }                                                    \
                break;                                               \
        }                                                            \
    } while (0)

inline int rows_per_block(int wpr) { return wpr <= 4 ? 4 / wpr : 1; }

// Grid and turns per row group. One row per group is the default: walking several rows per group
// (so that gamma / beta are fetched once per group) was measured at fp32 [8192,4096] over rotating
// buffers and lost more streaming rate than the saved vector traffic gave back (softmax 0.76 ->
// 0.72, RMSNorm 0.75 -> 0.74, LayerNorm 0.66 -> 0.68 of the HBM peak at 2 to 16 rows per group).
inline void row_launch_shape(int64_t rows, int wpr, int64_t &grid, int &iters) {
    static const int max_iters = [] {
        const char *e = std::getenv("FT_HIP_ROW_ITERS");  // tuning knob: most rows one row group walks (1 = one row per group)
        const int v = e ? std::atoi(e) : 1;
        return v < 1 ? 1 : v;
    }();
    const int cus = fth::compute_units() > 0 ? fth::compute_units() : 256;
    const int64_t resident_groups = (int64_t)cus * (2048 / (kWave * wpr));
    int64_t it = rows / resident_groups;
    it = it < 1 ? 1 : it > max_iters ? max_iters : it;
    grid = fth::ceil_div(fth::ceil_div(rows, it), rows_per_block(wpr));
    iters = (int)fth::ceil_div(rows, grid * rows_per_block(wpr));
}

template <typename T>
int32_t launch_softmax(const T *x, T *y, int64_t rows, int64_t cols, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(rows >= 0 && cols >= 0, "softmax: negative extent");
    if (rows == 0 || cols == 0) return FTH_OK;
    FTH_ARG(x && y, "softmax: NULL operand");
    hipStream_t st = fth::resolve_stream(s);
    constexpr int EPV = Vec128<T>::n;
    int vpl, wpr, iters = 1;
    int64_t grid = 0;
    if (cols % EPV == 0 && aligned16(x) && aligned16(y) && pick_row_shape(cols / EPV, 16, vpl, wpr) &&
        (row_launch_shape(rows, wpr, grid, iters), grid <= kMaxGrid)) {
        if (try_row_walk<T, RowOp::Softmax>(x, nullptr, nullptr, y, rows, cols, T(0), vpl, wpr, st)) {
            FTH_CHECK_LAUNCH("softmax");
            return FTH_OK;
        }
#define L(V_, W_) softmax_row_kernel<T, V_, W_><<<dim3((unsigned)grid), dim3(RowBlock<W_>::kThreads), 0, st>>>(x, y, rows, (int)cols, iters)
        FTH_ROW_DISPATCH(vpl, wpr, L);
#undef L
    } else {
        FTH_ARG(rows <= kMaxGrid, "softmax: too many rows for one launch");
        // odd lengths, unaligned rows and rows beyond 8192 vectors (a vocabulary): still one read and one write while the
        // row fits a workgroup's registers and LDS; only beyond that the three-sweep kernel
        if (!fth::softmax_resident_rows(x, y, rows, cols, st))
            softmax_stream_kernel<T><<<dim3((unsigned)rows), dim3(kBlock), 0, st>>>(x, y, rows, cols);
    }
    FTH_CHECK_LAUNCH("softmax");
    return FTH_OK;
}

template <typename T>
int32_t launch_softmax_strided(const T *x, T *y, int64_t outer, int64_t reduce, int64_t inner, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(outer >= 0 && reduce >= 0 && inner >= 0, "softmax: negative extent");
    if (outer == 0 || reduce == 0 || inner == 0) return FTH_OK;
    if (inner == 1) return launch_softmax<T>(x, y, outer, reduce, s);
    FTH_ARG(x && y, "softmax: NULL operand");
    int64_t grid = fth::ceil_div(outer * inner, kBlock);
    FTH_ARG(grid <= kMaxGrid, "softmax: too many lanes for one launch");
    softmax_strided_kernel<T><<<dim3((unsigned)grid), dim3(kBlock), 0, fth::resolve_stream(s)>>>(x, y, outer, reduce, inner);
    FTH_CHECK_LAUNCH("softmax_strided");
    return FTH_OK;
}

template <typename T, bool ADD>
int32_t launch_layernorm(const T *x, const T *x2, const T *w, const T *b, T *y, int64_t rows, int64_t cols,
                         T eps, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(rows >= 0 && cols >= 0, "layer_norm: negative extent");
    if (rows == 0 || cols == 0) return FTH_OK;
    FTH_ARG(x && y && (!ADD || x2), "layer_norm: NULL operand");
    hipStream_t st = fth::resolve_stream(s);
    constexpr int EPV = Vec128<T>::n;
    int vpl, wpr, iters = 1;
    int64_t grid = 0;
    bool vec_ok = cols % EPV == 0 && aligned16(x) && aligned16(y) && (!ADD || aligned16(x2)) &&
                  (!w || aligned16(w)) && (!b || aligned16(b));
    if (vec_ok && pick_row_shape(cols / EPV, ADD ? 8 : 16, vpl, wpr) && (row_launch_shape(rows, wpr, grid, iters), grid <= kMaxGrid)) {
        if constexpr (!ADD) {
            if (try_row_walk<T, RowOp::LayerNorm>(x, w, b, y, rows, cols, eps, vpl, wpr, st)) {
                FTH_CHECK_LAUNCH("layer_norm");
                return FTH_OK;
            }
            // (Three 512-thread workgroups per compute unit, which is what the kernel's 65 registers allow, stream best at
            // this shape: compiled for 64 registers and four per unit 0.704 of the HBM peak against 0.721, held to two 0.675.)
            // Two rows side by side (gamma / beta once per pair) where a lane's share of a row is at most four vectors and
            // there are rows enough to fill the chip that way; FT_HIP_LN_SIDE=0 keeps one row per group. Measured at fp32
            // [8192,4096] on rotating buffers: LayerNorm 0.70 -> 0.72 of the HBM peak with two rows, 0.64 with four (too few,
            // too fat workgroups); without gamma and beta one row per group streams best (0.76 against 0.72), and so it does for
            // RMSNorm with its single gamma (0.74 against 0.72 with two rows). At eight wavefronts per row (two vectors a
            // lane) three rows side by side measure 0.696 and four 0.659 against 0.722 with two. Across all variants the
            // rate follows the bytes a row moves from L2 into the compute unit: 16 KiB (softmax) 0.776, 32 KiB (RMSNorm;
            // LayerNorm two rows at a time) 0.72-0.76, 48 KiB (LayerNorm one row at a time) 0.67.
            constexpr int kSide = 2;
            static const bool side_off = [] {
                const char *e = std::getenv("FT_HIP_LN_SIDE");
                return e && std::atoi(e) == 0;
            }();
            const int cus = fth::compute_units() > 0 ? fth::compute_units() : 256;
            const int64_t side_grid = fth::ceil_div(rows, (int64_t)rows_per_block(wpr) * kSide);
            if ((w || b) && !side_off && iters == 1 && wpr <= 8 && vpl <= 4 && side_grid >= 4 * (int64_t)cus) {
#define LS(V_, W_) layernorm_rows_kernel<T, V_, W_, kSide><<<dim3((unsigned)side_grid), dim3(RowBlock<W_>::kThreads), 0, st>>>(x, w, b, y, rows, (int)cols, eps)
                switch (wpr) {
                    case 1: if (vpl == 1) { LS(1, 1); } else if (vpl == 2) { LS(2, 1); } else { LS(4, 1); } break;
                    case 2: if (vpl == 1) { LS(1, 2); } else if (vpl == 2) { LS(2, 2); } else { LS(4, 2); } break;
                    case 8: if (vpl == 1) { LS(1, 8); } else if (vpl == 2) { LS(2, 8); } else { LS(4, 8); } break;
                    default: if (vpl == 1) { LS(1, 4); } else if (vpl == 2) { LS(2, 4); } else { LS(4, 4); } break;
                }
#undef LS
                FTH_CHECK_LAUNCH("layer_norm");
                return FTH_OK;
            }
        }
#define L(V_, W_) layernorm_row_kernel<T, V_, W_, ADD><<<dim3((unsigned)grid), dim3(RowBlock<W_>::kThreads), 0, st>>>(x, x2, w, b, y, rows, (int)cols, eps, iters)
        FTH_ROW_DISPATCH(vpl, wpr, L);
#undef L
    } else {
        FTH_ARG(rows <= kMaxGrid, "layer_norm: too many rows for one launch");
        layernorm_stream_kernel<T, ADD><<<dim3((unsigned)rows), dim3(kBlock), 0, st>>>(x, x2, w, b, y, rows, cols, eps);
    }
    FTH_CHECK_LAUNCH("layer_norm");
    return FTH_OK;
}

template <typename T>
int32_t launch_rmsnorm(const T *x, const T *w, T *y, int64_t rows, int64_t cols, T eps, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(rows >= 0 && cols >= 0, "rms_norm: negative extent");
    if (rows == 0 || cols == 0) return FTH_OK;
    FTH_ARG(x && y, "rms_norm: NULL operand");
    hipStream_t st = fth::resolve_stream(s);
    constexpr int EPV = Vec128<T>::n;
    int vpl, wpr, iters = 1;
    int64_t grid = 0;
    if (cols % EPV == 0 && aligned16(x) && aligned16(y) && (!w || aligned16(w)) &&
        pick_row_shape(cols / EPV, 16, vpl, wpr) && (row_launch_shape(rows, wpr, grid, iters), grid <= kMaxGrid)) {
        // 512-thread workgroups with a gamma vector stream best three to a compute unit, as the two-row LayerNorm kernel does
        // by its registers (measured at fp32 [8192, 4096] on rotating buffers: four per unit 0.744 of the HBM peak, three 0.759,
        // two 0.733; softmax, which reads no second vector, is best at four). The kernel's registers would allow four, so 48 KiB
        // of unused dynamic LDS per workgroup hold the count at three.
        if (try_row_walk<T, RowOp::RmsNorm>(x, w, nullptr, y, rows, cols, eps, vpl, wpr, st)) {
            FTH_CHECK_LAUNCH("rms_norm");
            return FTH_OK;
        }
        const size_t pad = (wpr == 8 && w) ? (size_t)48 * 1024 : 0;
#define L(V_, W_) rmsnorm_row_kernel<T, V_, W_><<<dim3((unsigned)grid), dim3(RowBlock<W_>::kThreads), pad, st>>>(x, w, y, rows, (int)cols, eps, iters)
        FTH_ROW_DISPATCH(vpl, wpr, L);
#undef L
    } else {
        FTH_ARG(rows <= kMaxGrid, "rms_norm: too many rows for one launch");
        rmsnorm_stream_kernel<T><<<dim3((unsigned)rows), dim3(kBlock), 0, st>>>(x, w, y, rows, cols, eps);
    }
    FTH_CHECK_LAUNCH("rms_norm");
    return FTH_OK;
}

template <typename T, Ew OP>
int32_t launch_elementwise(const T *a, const T *b, T *y, int64_t n, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(n >= 0, "elementwise: negative length");
    if (n == 0) return FTH_OK;
    FTH_ARG(a && y && (OP != Ew::Add || b), "elementwise: NULL operand");
    hipStream_t st = fth::resolve_stream(s);
    constexpr int EPV = Vec128<T>::n;
    int64_t done = 0;
    if (aligned16(a) && aligned16(y) && (OP != Ew::Add || aligned16(b))) {
        int64_t nvec = n / EPV;
        if (nvec > 0) {
            static const int shape = [] {
                const char *e = std::getenv("FT_HIP_EW_SHAPE");  // tuning knob: 100 * vectors per thread + block threads / 64
                return e ? std::atoi(e) : 108;  // one vector per thread, 512-thread blocks: GELU at fp32 [8192,4096] 0.762 -> 0.784 of the HBM peak against 1024-thread blocks
            }();
            const int unr = shape / 100, bt = (shape % 100) * 64;
            int64_t grid = fth::ceil_div(nvec, (int64_t)bt * unr);
            FTH_ARG(grid <= kMaxGrid, "elementwise: too long for one launch");
            if (unr == 4 && bt == 256) elementwise_vec_kernel<T, OP, 4, 256><<<dim3((unsigned)grid), dim3(256), 0, st>>>(a, b, y, nvec);
            else if (unr == 1 && bt == 256) elementwise_vec_kernel<T, OP, 1, 256><<<dim3((unsigned)grid), dim3(256), 0, st>>>(a, b, y, nvec);
            else if (unr == 2 && bt == 1024) elementwise_vec_kernel<T, OP, 2, 1024><<<dim3((unsigned)grid), dim3(1024), 0, st>>>(a, b, y, nvec);
            else if (unr == 1 && bt == 512) elementwise_vec_kernel<T, OP, 1, 512><<<dim3((unsigned)grid), dim3(512), 0, st>>>(a, b, y, nvec);
            else {
                grid = fth::ceil_div(nvec, 1024);
                elementwise_vec_kernel<T, OP, 1, 1024><<<dim3((unsigned)grid), dim3(1024), 0, st>>>(a, b, y, nvec);
            }
            FTH_CHECK_LAUNCH("elementwise_vec");
        }
        done = nvec * EPV;
    }
    if (done < n) {
        int64_t grid = fth::ceil_div(n - done, kBlock);
        FTH_ARG(grid <= kMaxGrid, "elementwise: too long for one launch");
        elementwise_scalar_kernel<T, OP><<<dim3((unsigned)grid), dim3(kBlock), 0, st>>>(a, b, y, done, n);
        FTH_CHECK_LAUNCH("elementwise_scalar");
    }
    return FTH_OK;
}

template <typename T, bool RES>
int32_t launch_bias(const T *x, const T *bias, const T *res, T *y, int64_t rows, int64_t cols, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(rows >= 0 && cols >= 0, "bias_add: negative extent");
    if (rows == 0 || cols == 0) return FTH_OK;
    FTH_ARG(x && bias && y && (!RES || res), "bias_add: NULL operand");
    hipStream_t st = fth::resolve_stream(s);
    constexpr int EPV = Vec128<T>::n;
    int64_t total;
    if (cols % EPV == 0 && cols <= 2147483647LL && aligned16(x) && aligned16(bias) && aligned16(y) && (!RES || aligned16(res)) &&
        !__builtin_mul_overflow(rows, cols / EPV, &total) && fth::ceil_div(total, 256) <= kMaxGrid) {
        static const int bt = [] {
            const char *e = std::getenv("FT_HIP_BIAS_BLOCK");  // tuning knob: threads per block (256, 512 or 1024)
            return e ? std::atoi(e) : 512;  // (bias + residual at fp32 [8192,4096]: 0.785 of the HBM peak against 0.779 with 1024)
        }();
        if (bt == 256)
            bias_flat_kernel<T, RES, 256><<<dim3((unsigned)fth::ceil_div(total, 256)), dim3(256), 0, st>>>(x, bias, res, y, total, (int)(cols / EPV));
        else if (bt == 512)
            bias_flat_kernel<T, RES, 512><<<dim3((unsigned)fth::ceil_div(total, 512)), dim3(512), 0, st>>>(x, bias, res, y, total, (int)(cols / EPV));
        else
            bias_flat_kernel<T, RES, 1024><<<dim3((unsigned)fth::ceil_div(total, 1024)), dim3(1024), 0, st>>>(x, bias, res, y, total, (int)(cols / EPV));
    } else {
        int64_t grid = fth::ceil_div(rows * cols, kBlock);
        FTH_ARG(grid <= kMaxGrid, "bias_add: too long for one launch");
        bias_scalar_kernel<T, RES><<<dim3((unsigned)grid), dim3(kBlock), 0, st>>>(x, bias, res, y, rows, cols);
    }
    FTH_CHECK_LAUNCH("bias_add");
    return FTH_OK;
}

}  // namespace

extern "C" {

int32_t fth_dev_softmax_lastdim_f32(const float *x, float *y, int64_t rows, int64_t cols, fth_stream s) {
    return launch_softmax<float>(x, y, rows, cols, s);
}
int32_t fth_dev_softmax_lastdim_f64(const double *x, double *y, int64_t rows, int64_t cols, fth_stream s) {
    return launch_softmax<double>(x, y, rows, cols, s);
}
int32_t fth_dev_softmax_strided_f32(const float *x, float *y, int64_t outer, int64_t reduce, int64_t inner, fth_stream s) {
    return launch_softmax_strided<float>(x, y, outer, reduce, inner, s);
}
int32_t fth_dev_softmax_strided_f64(const double *x, double *y, int64_t outer, int64_t reduce, int64_t inner, fth_stream s) {
    return launch_softmax_strided<double>(x, y, outer, reduce, inner, s);
}
int32_t fth_dev_layer_norm_f32(const float *x, const float *weight, const float *bias, float *y, int64_t batch,
                               int64_t norm_size, float eps, fth_stream s) {
    return launch_layernorm<float, false>(x, nullptr, weight, bias, y, batch, norm_size, eps, s);
}
int32_t fth_dev_layer_norm_f64(const double *x, const double *weight, const double *bias, double *y, int64_t batch,
                               int64_t norm_size, double eps, fth_stream s) {
    return launch_layernorm<double, false>(x, nullptr, weight, bias, y, batch, norm_size, eps, s);
}
int32_t fth_dev_add_layer_norm_f32(const float *a, const float *b, const float *weight, const float *bias, float *y,
                                   int64_t batch, int64_t norm_size, float eps, fth_stream s) {
    return launch_layernorm<float, true>(a, b, weight, bias, y, batch, norm_size, eps, s);
}
int32_t fth_dev_rms_norm_f32(const float *x, const float *weight, float *y, int64_t batch, int64_t norm_size,
                             float eps, fth_stream s) {
    return launch_rmsnorm<float>(x, weight, y, batch, norm_size, eps, s);
}
int32_t fth_dev_rms_norm_f64(const double *x, const double *weight, double *y, int64_t batch, int64_t norm_size,
                             double eps, fth_stream s) {
    return launch_rmsnorm<double>(x, weight, y, batch, norm_size, eps, s);
}
int32_t fth_dev_gelu_f32(const float *x, float *y, int64_t n, fth_stream s) {
    return launch_elementwise<float, Ew::Gelu>(x, nullptr, y, n, s);
}
int32_t fth_dev_gelu_f64(const double *x, double *y, int64_t n, fth_stream s) {
    return launch_elementwise<double, Ew::Gelu>(x, nullptr, y, n, s);
}
int32_t fth_dev_gelu_tanh_f32(const float *x, float *y, int64_t n, fth_stream s) {
    return launch_elementwise<float, Ew::GeluTanh>(x, nullptr, y, n, s);
}
int32_t fth_dev_gelu_tanh_f64(const double *x, double *y, int64_t n, fth_stream s) {
    return launch_elementwise<double, Ew::GeluTanh>(x, nullptr, y, n, s);
}
int32_t fth_dev_add_f32(const float *a, const float *b, float *y, int64_t n, fth_stream s) {
    return launch_elementwise<float, Ew::Add>(a, b, y, n, s);
}
int32_t fth_dev_add_f64(const double *a, const double *b, double *y, int64_t n, fth_stream s) {
    return launch_elementwise<double, Ew::Add>(a, b, y, n, s);
}
int32_t fth_dev_copy_f32(const float *x, float *y, int64_t n, fth_stream s) {
    return launch_elementwise<float, Ew::Copy>(x, nullptr, y, n, s);
}
int32_t fth_dev_copy_f64(const double *x, double *y, int64_t n, fth_stream s) {
    return launch_elementwise<double, Ew::Copy>(x, nullptr, y, n, s);
}
int32_t fth_dev_bias_add_f32(const float *x, const float *bias, float *y, int64_t rows, int64_t cols, fth_stream s) {
    return launch_bias<float, false>(x, bias, nullptr, y, rows, cols, s);
}
int32_t fth_dev_bias_add_f64(const double *x, const double *bias, double *y, int64_t rows, int64_t cols, fth_stream s) {
    return launch_bias<double, false>(x, bias, nullptr, y, rows, cols, s);
}
int32_t fth_dev_bias_residual_add_f32(const float *x, const float *bias, const float *residual, float *y,
                                      int64_t rows, int64_t cols, fth_stream s) {
    return launch_bias<float, true>(x, bias, residual, y, rows, cols, s);
}
int32_t fth_dev_bias_residual_add_f64(const double *x, const double *bias, const double *residual, double *y,
                                      int64_t rows, int64_t cols, fth_stream s) {
    return launch_bias<double, true>(x, bias, residual, y, rows, cols, s);
}

}  // extern "C"
