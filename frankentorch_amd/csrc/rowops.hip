// Memory-bound row kernels for gfx950: last-dim softmax, LayerNorm, add+LayerNorm, RMSNorm,
// erf-GELU, add, bias add, bias+residual add.
//
// Shape of every row kernel: one, two or four 64-lane wavefronts of a 256-thread block own one
// row (the fewest that keep a lane at <= 4 vectors; up to 16 vectors per lane for rows of up to
// 16 Ki elements), pull it from HBM once with 128-bit loads into registers, reduce with a fixed
// xor-butterfly over the wavefront and a fixed left-to-right fold over the row's wavefronts, and
// write the row back once with 128-bit non-temporal stores. No atomics anywhere: the reduction
// tree is a function of (row length, kernel variant) only, so repeated runs are bitwise
// identical. Rows whose base is not 16-byte aligned, whose length is not a multiple of the
// vector width, or which do not fit the register budget take a block-per-row streaming variant
// with the same fixed trees.
//
// Arithmetic follows crates/ft-kernel-cpu/src/lib.rs step for step (separate multiplies and adds;
// this file is compiled with -ffp-contract=off): softmax :39219-39229, LayerNorm :5886-5909,
// add+LayerNorm :5946-5970, RMSNorm :6466-6480, GELU :36966-36969, add :36870-36877,
// bias pass :17336-17351. Only the summation ORDER differs (tree instead of sequential /
// pairwise-128), which is what the 1e-5 tolerance of the parity tests covers.

#include <cstdlib>
#include <initializer_list>

#include "common.hpp"

namespace {

constexpr int kWave = 64;
constexpr int kBlock = 256;

// Streaming stores carry the non-temporal hint: an output is written once and not re-read by the
// kernel, so it should not displace the input (which a producer kernel may just have left in the
// last-level cache) or the reusable gamma / beta / bias lines. Loads stay temporal: measured on
// MI355X at fp32 [8192,4096], non-temporal loads cost 8-10 % on every kernel, non-temporal stores
// gain 2-25 %.
typedef float nat_f4 __attribute__((ext_vector_type(4)));
typedef double nat_d2 __attribute__((ext_vector_type(2)));
#ifndef FTH_NT_LOAD
#define FTH_NT_LOAD 0
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

// exp(x) = 2^(x * log2 e) on the hardware exp2 unit. The product x * log2 e is carried in two
// pieces (t + r, with the rounding error of the multiply recovered by an FMA and the low bits of
// log2 e added), and 2^r is folded back as 1 + r ln 2, so the result stays within about 1.5 ULP
// instead of the |x| * 2^-24 relative error of a bare exp2(x * log2e). -inf maps to exactly 0 and
// NaN propagates, which the softmax special cases rely on. Results below 2^-126 flush to zero.
__device__ __forceinline__ float dev_exp(float x) {
    const float kL2eHi = 1.44269502162933349609375f;  // float(log2 e)
    const float kL2eLo = 1.925963033500011e-8f;       // log2 e - float(log2 e)
    const float kLn2 = 0.693147182464599609375f;
    const float t = x * kL2eHi;
    float r = __builtin_fmaf(x, kL2eHi, -t);
    r = __builtin_fmaf(x, kL2eLo, r);
    r = (x == -__builtin_inff()) ? 0.0f : r;
    const float e = __builtin_amdgcn_exp2f(t);
    return __builtin_fmaf(e * r, kLn2, e);
}
__device__ __forceinline__ double dev_exp(double x) { return exp(x); }
__device__ __forceinline__ float dev_sqrt(float x) { return sqrtf(x); }
__device__ __forceinline__ double dev_sqrt(double x) { return sqrt(x); }
__device__ __forceinline__ float dev_max(float a, float b) { return fmaxf(a, b); }
__device__ __forceinline__ double dev_max(double a, double b) { return fmax(a, b); }
__device__ __forceinline__ float dev_gelu(float x) {
    return (0.5f * x) * (1.0f + erff(x * 0.70710678118654752440f));
}
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

// Reduction over the WPR wavefronts that share a row (WPR == 1: the wavefront alone; WPR == 2 or
// 4: the row's wavefronts inside the 256-thread block, folded left to right through LDS). Every
// thread of the block reaches the barriers (blocks with WPR > 1 never exit early).
template <int WPR, typename T, class F>
__device__ __forceinline__ T group_reduce(T v, F f, T *smem) {
    v = wave_reduce(v, f);
    if constexpr (WPR == 1) {
        return v;
    } else {
        const int wave = threadIdx.x / kWave;
        const int first = (wave / WPR) * WPR;
        __syncthreads();
        if ((threadIdx.x & (kWave - 1)) == 0) smem[wave] = v;
        __syncthreads();
        T r = smem[first];
#pragma unroll
        for (int w = 1; w < WPR; ++w) r = f(r, smem[first + w]);
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

// A 256-thread block holds 4 / WPR rows.
template <int WPR> __device__ __forceinline__ int64_t row_of_block() {
    return (int64_t)blockIdx.x * (kBlock / (kWave * WPR)) + threadIdx.x / (kWave * WPR);
}
// Rows past the end are clamped (so every wavefront still reaches the block barriers) and their
// stores are suppressed by passing nvec_store == 0.
#define FTH_ROW_PROLOGUE(WPR_)                                  \
    int64_t row = row_of_block<WPR_>();                         \
    const bool row_live = row < rows;                           \
    if constexpr (WPR_ == 1) {                                  \
        if (!row_live) return;                                  \
    } else {                                                    \
        if (!row_live) row = rows - 1;                          \
    }

// ---- softmax ------------------------------------------------------------------------------
template <typename T, int VPL, int WPR>
__global__ __launch_bounds__(kBlock) void softmax_row_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                             int64_t rows, int cols) {
    __shared__ T smem[4];
    using R = RowRegs<T, VPL, WPR>;
    FTH_ROW_PROLOGUE(WPR)
    const int nvec = cols / R::EPV;
    R r;
    r.load(x + row * cols, nvec, neg_inf<T>());
    T m = neg_inf<T>();
#pragma unroll
    for (int i = 0; i < VPL; ++i)
#pragma unroll
        for (int j = 0; j < R::EPV; ++j) m = dev_max(m, r.e[i][j]);
    m = group_reduce<WPR>(m, MaxOp{}, smem);
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
    s = group_reduce<WPR>(s, SumOp{}, smem);
    // One correctly rounded 1 / s per row, then a multiply per element (the reference divides each
    // element: the two differ by at most one rounding, far inside the parity tolerance, and the
    // per-element IEEE division sequence would make this kernel ALU-bound).
    const T inv = T(1) / s;
#pragma unroll
    for (int i = 0; i < VPL; ++i)
#pragma unroll
        for (int j = 0; j < R::EPV; ++j) r.e[i][j] = r.e[i][j] * inv;
    r.store(y + row * cols, row_live ? nvec : 0);
}

// ---- LayerNorm / add+LayerNorm ---------------------------------------------------------------
template <typename T, int VPL, int WPR, bool ADD>
__global__ __launch_bounds__(kBlock) void layernorm_row_kernel(const T *__restrict__ x, const T *__restrict__ x2,
                                                               const T *__restrict__ w, const T *__restrict__ b,
                                                               T *__restrict__ y, int64_t rows, int cols, T eps) {
    __shared__ T smem[4];
    using R = RowRegs<T, VPL, WPR>;
    FTH_ROW_PROLOGUE(WPR)
    const int nvec = cols / R::EPV;
    R r;
    r.load(x + row * cols, nvec, T(0));
    if constexpr (ADD) {
        R r2;
        r2.load(x2 + row * cols, nvec, T(0));
#pragma unroll
        for (int i = 0; i < VPL; ++i)
#pragma unroll
            for (int j = 0; j < R::EPV; ++j) r.e[i][j] = r.e[i][j] + r2.e[i][j];
    }
    const T inv_n = T(1) / (T)cols;
    T sum = 0;
#pragma unroll
    for (int i = 0; i < VPL; ++i)
#pragma unroll
        for (int j = 0; j < R::EPV; ++j) sum += r.e[i][j];
    sum = group_reduce<WPR>(sum, SumOp{}, smem);
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
    vsum = group_reduce<WPR>(vsum, SumOp{}, smem);
    const T rstd = T(1) / dev_sqrt(vsum * inv_n + eps);
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
        const int v = R::lane() + i * R::kLanes;
        if (v < nvec) {
            T wv[R::EPV], bv[R::EPV];
            if (w) R::load_vec(w, v, wv);
            if (b) R::load_vec(b, v, bv);
#pragma unroll
            for (int j = 0; j < R::EPV; ++j) {
                T o = (r.e[i][j] - mean) * rstd;
                if (w) o = o * wv[j];
                if (b) o = o + bv[j];
                r.e[i][j] = o;
            }
        }
    }
    r.store(y + row * cols, row_live ? nvec : 0);
}

// ---- RMSNorm ---------------------------------------------------------------------------------
template <typename T, int VPL, int WPR>
__global__ __launch_bounds__(kBlock) void rmsnorm_row_kernel(const T *__restrict__ x, const T *__restrict__ w,
                                                             T *__restrict__ y, int64_t rows, int cols, T eps) {
    __shared__ T smem[4];
    using R = RowRegs<T, VPL, WPR>;
    FTH_ROW_PROLOGUE(WPR)
    const int nvec = cols / R::EPV;
    R r;
    r.load(x + row * cols, nvec, T(0));
    const T inv_n = T(1) / (T)cols;
    T ss = 0;
#pragma unroll
    for (int i = 0; i < VPL; ++i)
#pragma unroll
        for (int j = 0; j < R::EPV; ++j) ss += r.e[i][j] * r.e[i][j];
    ss = group_reduce<WPR>(ss, SumOp{}, smem);
    const T rstd = T(1) / dev_sqrt(ss * inv_n + eps);
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
        const int v = R::lane() + i * R::kLanes;
        if (v < nvec) {
            T wv[R::EPV];
            if (w) R::load_vec(w, v, wv);
#pragma unroll
            for (int j = 0; j < R::EPV; ++j) {
                T o = r.e[i][j] * rstd;
                if (w) o = o * wv[j];
                r.e[i][j] = o;
            }
        }
    }
    r.store(y + row * cols, row_live ? nvec : 0);
}

// ---------------------------------------------------------------------------------------------
// Streaming variants: one 256-thread block per row, scalar loads, the row is re-read from L2.
// ---------------------------------------------------------------------------------------------
template <typename T, class F>
__device__ __forceinline__ T block_reduce(T v, F f, T *smem) {
    return group_reduce<4>(v, f, smem);
}

template <typename T>
__global__ __launch_bounds__(kBlock) void softmax_stream_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                                int64_t rows, int64_t cols) {
    __shared__ T smem[4];
    const T *xr = x + (int64_t)blockIdx.x * cols;
    T *yr = y + (int64_t)blockIdx.x * cols;
    T m = neg_inf<T>();
    for (int64_t j = threadIdx.x; j < cols; j += kBlock) m = dev_max(m, xr[j]);
    m = block_reduce(m, MaxOp{}, smem);
    T s = 0;
    for (int64_t j = threadIdx.x; j < cols; j += kBlock) {
        T ev = dev_exp(xr[j] - m);
        yr[j] = ev;
        s += ev;
    }
    s = block_reduce(s, SumOp{}, smem);
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
    __shared__ T smem[4];
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
    sum = block_reduce(sum, SumOp{}, smem);
    const T mean = sum * inv_n;
    const T *src = ADD ? yr : xr;
    T vsum = 0;
    for (int64_t j = threadIdx.x; j < cols; j += kBlock) {
        T d = src[j] - mean;
        vsum += d * d;
    }
    vsum = block_reduce(vsum, SumOp{}, smem);
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
    __shared__ T smem[4];
    const T *xr = x + (int64_t)blockIdx.x * cols;
    T *yr = y + (int64_t)blockIdx.x * cols;
    const T inv_n = T(1) / (T)cols;
    T ss = 0;
    for (int64_t j = threadIdx.x; j < cols; j += kBlock) ss += xr[j] * xr[j];
    ss = block_reduce(ss, SumOp{}, smem);
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
enum class Ew { Gelu, Add, GeluTanh };
constexpr int kUnr = 4;

template <typename T, Ew OP>
__global__ __launch_bounds__(kBlock) void elementwise_vec_kernel(const T *__restrict__ a, const T *__restrict__ b,
                                                                 T *__restrict__ y, int64_t nvec) {
    using R = RowRegs<T, 1, 1>;
    using V = typename Vec128<T>::type;
    const int64_t base = (int64_t)blockIdx.x * (kBlock * kUnr) + threadIdx.x;
    V va[kUnr], vb[kUnr];
#pragma unroll
    for (int u = 0; u < kUnr; ++u) {
        int64_t v = base + (int64_t)u * kBlock;
        if (v < nvec) {
            va[u] = stream_load(reinterpret_cast<const V *>(a) + v);
            if constexpr (OP == Ew::Add) vb[u] = stream_load(reinterpret_cast<const V *>(b) + v);
        }
    }
#pragma unroll
    for (int u = 0; u < kUnr; ++u) {
        int64_t v = base + (int64_t)u * kBlock;
        if (v < nvec) {
            T ea[R::EPV], eb[R::EPV];
            R::unpack(va[u], ea);
            if constexpr (OP == Ew::Add) R::unpack(vb[u], eb);
#pragma unroll
            for (int j = 0; j < R::EPV; ++j) {
                if constexpr (OP == Ew::Gelu) ea[j] = dev_gelu(ea[j]);
                else if constexpr (OP == Ew::GeluTanh) ea[j] = dev_gelu_tanh(ea[j]);
                else ea[j] = ea[j] + eb[j];
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
    else y[i] = a[i] + b[i];
}

// ---- bias add / bias + residual add: y[r, j] = (x[r, j] + bias[j]) (+ res[r, j]) --------------
// One wavefront per row so the bias index is the vector index (no division).
template <typename T, bool RES>
__global__ __launch_bounds__(kBlock) void bias_row_kernel(const T *x, const T *__restrict__ bias,
                                                          const T *res, T *y, int64_t rows, int cols) {
    using R = RowRegs<T, 1, 1>;
    using V = typename Vec128<T>::type;
    const int64_t row = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
    if (row >= rows) return;
    const int lane = threadIdx.x & (kWave - 1);
    const int nvec = cols / R::EPV;
    const V *xr = reinterpret_cast<const V *>(x + row * cols);
    const V *rr = RES ? reinterpret_cast<const V *>(res + row * cols) : nullptr;
    const V *br = reinterpret_cast<const V *>(bias);
    V *yr = reinterpret_cast<V *>(y + row * cols);
    for (int v0 = lane; v0 < nvec; v0 += kWave * kUnr) {
        V vx[kUnr], vr[kUnr], vb[kUnr];
#pragma unroll
        for (int u = 0; u < kUnr; ++u) {
            int v = v0 + u * kWave;
            if (v < nvec) {
                vx[u] = stream_load(xr + v);
                vb[u] = br[v];
                if constexpr (RES) vr[u] = stream_load(rr + v);
            }
        }
#pragma unroll
        for (int u = 0; u < kUnr; ++u) {
            int v = v0 + u * kWave;
            if (v < nvec) {
                T ex[R::EPV], eb[R::EPV], er[R::EPV];
                R::unpack(vx[u], ex);
                R::unpack(vb[u], eb);
                if constexpr (RES) R::unpack(vr[u], er);
#pragma unroll
                for (int j = 0; j < R::EPV; ++j) {
                    T o = ex[j] + eb[j];
                    if constexpr (RES) o = o + er[j];
                    ex[j] = o;
                }
                stream_store(yr + v, R::pack(ex));
            }
        }
    }
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

// Picks (VPL, WPR) for a register-resident row of `nvec` vectors, or returns false.
// Few vectors per lane and more wavefronts per row measured best on MI355X (fp32 [8192,4096]:
// LayerNorm 74 % of HBM peak with 16 vectors x 1 wavefront, 85 % with 4 x 4), so the row is spread
// over the fewest wavefronts that keep a lane at <= 4 vectors, and only longer rows grow the
// per-lane count. `max_vpl` caps the vectors a lane may hold.
inline bool pick_row_shape(int64_t nvec, int max_vpl, int &vpl, int &wpr) {
    if (nvec <= 0 || nvec > 256 * (int64_t)max_vpl) return false;
    static const int forced = [] {
        const char *e = std::getenv("FT_HIP_ROW_WPR");  // tuning knob: wavefronts per row (1, 2 or 4)
        return e ? std::atoi(e) : 0;
    }();
    int w = nvec <= 64 * 4 ? 1 : nvec <= 128 * 4 ? 2 : 4;
    if (forced == 1 || forced == 2 || forced == 4) {
        if (fth::ceil_div(nvec, 64 * forced) <= max_vpl) w = forced;
    }
    const int64_t need = fth::ceil_div(nvec, 64 * w);
    int v = need <= 1 ? 1 : need <= 2 ? 2 : need <= 4 ? 4 : need <= 8 ? 8 : 16;
    // instantiated shapes: WPR 1 x {1,2,4,8,16}, WPR 2 x {4,8,16}, WPR 4 x {2,4,8,16}
    if (w == 2 && v < 4) v = 4;
    if (w == 4 && v < 2) v = 2;
    vpl = v;
    wpr = w;
    return true;
}

#define FTH_ROW_DISPATCH(VPL_, WPR_, LAUNCH)                         \
    do {                                                             \
        if (WPR_ == 1) {                                             \
            switch (VPL_) {                                          \
                case 1: { LAUNCH(1, 1); } break;                     \
                case 2: { LAUNCH(2, 1); } break;                     \
                case 4: { LAUNCH(4, 1); } break;                     \
                case 8: { LAUNCH(8, 1); } break;                     \
                default: { LAUNCH(16, 1); } break;                   \
            }                                                        \
        } else if (WPR_ == 2) {                                      \
            switch (VPL_) {                                          \
                case 4: { LAUNCH(4, 2); } break;                     \
                case 8: { LAUNCH(8, 2); } break;                     \
                default: { LAUNCH(16, 2); } break;                   \
            }                                                        \
        } else {                                                     \
            switch (VPL_) {                                          \
                case 2: { LAUNCH(2, 4); } break;                     \
                case 4: { LAUNCH(4, 4); } break;                     \
                case 8: { LAUNCH(8, 4); } break;                     \
                default: { LAUNCH(16, 4); } break;                   \
            }                                                        \
        }                                                            \
    } while (0)

inline int64_t row_grid(int64_t rows, int wpr) { return fth::ceil_div(rows, 4 / wpr); }

template <typename T>
int32_t launch_softmax(const T *x, T *y, int64_t rows, int64_t cols, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(rows >= 0 && cols >= 0, "softmax: negative extent");
    if (rows == 0 || cols == 0) return FTH_OK;
    FTH_ARG(x && y, "softmax: NULL operand");
    hipStream_t st = fth::resolve_stream(s);
    constexpr int EPV = Vec128<T>::n;
    int vpl, wpr;
    if (cols % EPV == 0 && aligned16(x) && aligned16(y) && pick_row_shape(cols / EPV, 16, vpl, wpr) &&
        row_grid(rows, wpr) <= kMaxGrid) {
#define L(V_, W_) softmax_row_kernel<T, V_, W_><<<dim3((unsigned)row_grid(rows, W_)), dim3(kBlock), 0, st>>>(x, y, rows, (int)cols)
        FTH_ROW_DISPATCH(vpl, wpr, L);
#undef L
    } else {
        FTH_ARG(rows <= kMaxGrid, "softmax: too many rows for one launch");
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
    int vpl, wpr;
    bool vec_ok = cols % EPV == 0 && aligned16(x) && aligned16(y) && (!ADD || aligned16(x2)) &&
                  (!w || aligned16(w)) && (!b || aligned16(b));
    if (vec_ok && pick_row_shape(cols / EPV, 16, vpl, wpr) && row_grid(rows, wpr) <= kMaxGrid) {
#define L(V_, W_) layernorm_row_kernel<T, V_, W_, ADD><<<dim3((unsigned)row_grid(rows, W_)), dim3(kBlock), 0, st>>>(x, x2, w, b, y, rows, (int)cols, eps)
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
    int vpl, wpr;
    if (cols % EPV == 0 && aligned16(x) && aligned16(y) && (!w || aligned16(w)) &&
        pick_row_shape(cols / EPV, 16, vpl, wpr) && row_grid(rows, wpr) <= kMaxGrid) {
#define L(V_, W_) rmsnorm_row_kernel<T, V_, W_><<<dim3((unsigned)row_grid(rows, W_)), dim3(kBlock), 0, st>>>(x, w, y, rows, (int)cols, eps)
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
            int64_t grid = fth::ceil_div(nvec, kBlock * kUnr);
            FTH_ARG(grid <= kMaxGrid, "elementwise: too long for one launch");
            elementwise_vec_kernel<T, OP><<<dim3((unsigned)grid), dim3(kBlock), 0, st>>>(a, b, y, nvec);
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
    if (cols % EPV == 0 && cols <= 2147483647LL && aligned16(x) && aligned16(bias) && aligned16(y) &&
        (!RES || aligned16(res)) && fth::ceil_div(rows, 4) <= kMaxGrid) {
        bias_row_kernel<T, RES><<<dim3((unsigned)fth::ceil_div(rows, 4)), dim3(kBlock), 0, st>>>(x, bias, res, y, rows, (int)cols);
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
