// log-softmax and the fused softmax-cross-entropy loss (forward and backward) for gfx950.
//
// replaces log_softmax_dim_tensor_contiguous_f32 / _f64 (crates/ft-kernel-cpu/src/lib.rs:39298-39375,
// 18504-18590), cross_entropy_forward_f32 / _f64 (:6717-6738, 6649-6671) and
// cross_entropy_backward_f32 / _f64 (:6745-6781, 6679-6712).
//
// All three are HBM-bound row passes over [rows, classes] logits whose rows (50 257 floats for the
// GPT-2 vocabulary) are neither a vector multiple nor aligned, so a 256-thread workgroup owns one
// row and streams it with coalesced scalar loads; the second and third sweeps of a row hit L2.
// Reductions are a fixed butterfly per wavefront and a fixed fold across the four wavefronts
// (the reference scans a row sequentially; same values re-associated, inside the parity
// tolerance), so results are bitwise repeatable. Class indices arrive as int64; an index outside
// [0, classes) (the reference would panic on the slice index) is reported through `bad_index` as
// the lowest offending row, and that row's outputs are left unwritten.

#include "common.hpp"

namespace {

constexpr int kWave = 64;
constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;

template <typename T> __device__ __forceinline__ T t_exp(T v);
template <> __device__ __forceinline__ float t_exp<float>(float v) { return expf(v); }
template <> __device__ __forceinline__ double t_exp<double>(double v) { return exp(v); }
template <typename T> __device__ __forceinline__ T t_log(T v);
template <> __device__ __forceinline__ float t_log<float>(float v) { return logf(v); }
template <> __device__ __forceinline__ double t_log<double>(double v) { return log(v); }

// max that skips NaN operands the way f32::max / f64::max do (the reference's fold for log-softmax).
template <typename T> __device__ __forceinline__ T max_num(T a, T b) {
    if (a != a) return b;
    if (b != b) return a;
    return a > b ? a : b;
}
// the strict `>` scan of the cross-entropy kernels: a NaN never replaces the running maximum
template <typename T> __device__ __forceinline__ T max_gt(T a, T b) { return b > a ? b : a; }

template <typename T, class F> __device__ __forceinline__ T block_reduce(T v, F f, T *red, int &phase) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = f(v, __shfl_xor(v, off, kWave));
    T *buf = red + phase * kWaves;  // alternate halves: one barrier per reduction is enough
    phase ^= 1;
    if (lane == 0) buf[wave] = v;
    __syncthreads();
    T s = buf[0];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) s = f(s, buf[w]);
    return s;
}
struct SumOp {
    template <typename T> __device__ __forceinline__ T operator()(T a, T b) const { return a + b; }
};
struct MaxNumOp {
    template <typename T> __device__ __forceinline__ T operator()(T a, T b) const { return max_num(a, b); }
};
struct MaxGtOp {
    template <typename T> __device__ __forceinline__ T operator()(T a, T b) const { return max_gt(a, b); }
};

// out = (x - max) - ln(sum exp(x - max)) over a contiguous row.
template <typename T>
__global__ __launch_bounds__(kThreads) void log_softmax_rows_kernel(const T *__restrict__ x, T *__restrict__ y, int64_t cols) {
    __shared__ T red[2 * kWaves];
    int phase = 0;
    const T *xr = x + (int64_t)blockIdx.x * cols;
    T *yr = y + (int64_t)blockIdx.x * cols;
    T m = -__builtin_inf();
    for (int64_t j = threadIdx.x; j < cols; j += kThreads) m = max_num(m, xr[j]);
    m = block_reduce(m, MaxNumOp{}, red, phase);
    T s = T(0);
    for (int64_t j = threadIdx.x; j < cols; j += kThreads) s += t_exp<T>(xr[j] - m);
    s = block_reduce(s, SumOp{}, red, phase);
    const T lse = t_log<T>(s);
    for (int64_t j = threadIdx.x; j < cols; j += kThreads) yr[j] = (xr[j] - m) - lse;
}

// log-softmax over the middle dim of [outer, reduce, inner]: one thread per (outer, inner) lane,
// coalesced along inner, sequential over reduce.
template <typename T>
__global__ __launch_bounds__(kThreads) void log_softmax_strided_kernel(const T *__restrict__ x, T *__restrict__ y, int64_t outer,
                                                                      int64_t reduce, int64_t inner) {
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= outer * inner) return;
    const int64_t o = idx / inner, in = idx % inner;
    const T *xb = x + o * reduce * inner + in;
    T *yb = y + o * reduce * inner + in;
    T m = -__builtin_inf();
    for (int64_t r = 0; r < reduce; ++r) m = max_num(m, xb[r * inner]);
    T s = T(0);
    for (int64_t r = 0; r < reduce; ++r) s += t_exp<T>(xb[r * inner] - m);
    const T lse = t_log<T>(s);
    for (int64_t r = 0; r < reduce; ++r) yb[r * inner] = (xb[r * inner] - m) - lse;
}

// Row statistics shared by the two cross-entropy kernels: m (strict max scan) and s = sum exp(v - m).
template <typename T> __device__ __forceinline__ void ce_row_stats(const T *row, int64_t classes, T *red, int &phase, T &m, T &s) {
    m = -__builtin_inf();
    for (int64_t c = threadIdx.x; c < classes; c += kThreads) m = max_gt(m, row[c]);
    m = block_reduce(m, MaxGtOp{}, red, phase);
    s = T(0);
    for (int64_t c = threadIdx.x; c < classes; c += kThreads) s += t_exp<T>(row[c] - m);
    s = block_reduce(s, SumOp{}, red, phase);
}

__device__ __forceinline__ void note_bad(int64_t *bad_index, int64_t row) {
    if (bad_index && threadIdx.x == 0) atomicMin(reinterpret_cast<unsigned long long *>(bad_index), (unsigned long long)row);
}

template <typename T>
__global__ __launch_bounds__(kThreads) void cross_entropy_forward_kernel(const T *__restrict__ logits, const int64_t *__restrict__ target,
                                                                        int64_t classes, T *__restrict__ loss, int64_t *bad_index) {
    __shared__ T red[2 * kWaves];
    int phase = 0;
    const int64_t i = blockIdx.x;
    const int64_t t = target[i];
    if (t < 0 || t >= classes) {  // uniform over the workgroup
        note_bad(bad_index, i);
        return;
    }
    const T *row = logits + i * classes;
    T m, s;
    ce_row_stats(row, classes, red, phase, m, s);
    if (threadIdx.x == 0) loss[i] = (m + t_log<T>(s)) - row[t];
}

template <typename T>
__global__ __launch_bounds__(kThreads) void cross_entropy_backward_kernel(const T *__restrict__ logits, const int64_t *__restrict__ target,
                                                                         const T *__restrict__ dloss, int64_t classes,
                                                                         T *__restrict__ dlogits, int64_t *bad_index) {
    __shared__ T red[2 * kWaves];
    int phase = 0;
    const int64_t i = blockIdx.x;
    const int64_t t = target[i];
    if (t < 0 || t >= classes) {
        note_bad(bad_index, i);
        return;
    }
    const T *row = logits + i * classes;
    T *drow = dlogits + i * classes;
    T m, s;
    ce_row_stats(row, classes, red, phase, m, s);
    const T lse = m + t_log<T>(s), g = dloss[i];
    for (int64_t c = threadIdx.x; c < classes; c += kThreads) drow[c] = g * (t_exp<T>(row[c] - lse) - (c == t ? T(1) : T(0)));
}

__global__ void set_bad_index_kernel(int64_t *bad_index) { *bad_index = 0x7FFFFFFFFFFFFFFFLL; }
__global__ void finish_bad_index_kernel(int64_t *bad_index) {
    if (*bad_index == 0x7FFFFFFFFFFFFFFFLL) *bad_index = -1;
}

template <typename T> int32_t log_softmax_entry(const T *x, T *y, int64_t outer, int64_t reduce, int64_t inner, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(outer >= 0 && reduce >= 0 && inner >= 0, "log_softmax: negative extent");
    if (outer == 0 || reduce == 0 || inner == 0) return FTH_OK;
    FTH_ARG(x && y, "log_softmax: NULL operand");
    hipStream_t st = fth::resolve_stream(s);
    if (inner == 1) {
        FTH_ARG(outer <= 2147483647LL, "log_softmax: too many rows for one launch");
        log_softmax_rows_kernel<T><<<dim3((unsigned)outer), dim3(kThreads), 0, st>>>(x, y, reduce);
    } else {
        int64_t lanes;
        FTH_ARG(!__builtin_mul_overflow(outer, inner, &lanes) && fth::ceil_div(lanes, kThreads) <= 2147483647LL,
                "log_softmax: too many lanes for one launch");
        log_softmax_strided_kernel<T><<<dim3((unsigned)fth::ceil_div(lanes, kThreads)), dim3(kThreads), 0, st>>>(x, y, outer, reduce, inner);
    }
    FTH_CHECK_LAUNCH("log_softmax");
    return FTH_OK;
}

template <typename T>
int32_t cross_entropy_entry(bool backward, const T *logits, const int64_t *target, const T *dloss, int64_t batch, int64_t classes, T *out,
                            int64_t *bad_index, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(batch >= 0 && classes >= 0, "cross_entropy: negative extent");
    hipStream_t st = fth::resolve_stream(s);
    if (bad_index) {
        set_bad_index_kernel<<<1, 1, 0, st>>>(bad_index);
        FTH_CHECK_LAUNCH("cross_entropy_bad_index");
    }
    if (batch > 0) {
        FTH_ARG(logits && target && out && (!backward || dloss), "cross_entropy: NULL operand");
        FTH_ARG(batch <= 2147483647LL, "cross_entropy: too many rows for one launch");
        if (backward)
            cross_entropy_backward_kernel<T><<<dim3((unsigned)batch), dim3(kThreads), 0, st>>>(logits, target, dloss, classes, out, bad_index);
        else
            cross_entropy_forward_kernel<T><<<dim3((unsigned)batch), dim3(kThreads), 0, st>>>(logits, target, classes, out, bad_index);
        FTH_CHECK_LAUNCH("cross_entropy");
    }
    if (bad_index) {
        finish_bad_index_kernel<<<1, 1, 0, st>>>(bad_index);
        FTH_CHECK_LAUNCH("cross_entropy_bad_index");
    }
    return FTH_OK;
}

}  // namespace

extern "C" {

int32_t fth_dev_log_softmax_strided_f32(const float *x, float *y, int64_t outer, int64_t reduce, int64_t inner, fth_stream s) {
    return log_softmax_entry<float>(x, y, outer, reduce, inner, s);
}
int32_t fth_dev_log_softmax_strided_f64(const double *x, double *y, int64_t outer, int64_t reduce, int64_t inner, fth_stream s) {
    return log_softmax_entry<double>(x, y, outer, reduce, inner, s);
}
int32_t fth_dev_cross_entropy_forward_f32(const float *logits, const int64_t *target, int64_t batch, int64_t classes, float *loss,
                                          int64_t *bad_index, fth_stream s) {
    return cross_entropy_entry<float>(false, logits, target, nullptr, batch, classes, loss, bad_index, s);
}
int32_t fth_dev_cross_entropy_forward_f64(const double *logits, const int64_t *target, int64_t batch, int64_t classes, double *loss,
                                          int64_t *bad_index, fth_stream s) {
    return cross_entropy_entry<double>(false, logits, target, nullptr, batch, classes, loss, bad_index, s);
}
int32_t fth_dev_cross_entropy_backward_f32(const float *logits, const int64_t *target, const float *dloss, int64_t batch, int64_t classes,
                                           float *dlogits, int64_t *bad_index, fth_stream s) {
    return cross_entropy_entry<float>(true, logits, target, dloss, batch, classes, dlogits, bad_index, s);
}
int32_t fth_dev_cross_entropy_backward_f64(const double *logits, const int64_t *target, const double *dloss, int64_t batch, int64_t classes,
                                           double *dlogits, int64_t *bad_index, fth_stream s) {
    return cross_entropy_entry<double>(true, logits, target, dloss, batch, classes, dlogits, bad_index, s);
}

}  // extern "C"
