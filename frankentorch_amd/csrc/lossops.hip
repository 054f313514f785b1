// log-softmax and the fused softmax-cross-entropy loss (forward and backward) for gfx950.
//
// replaces log_softmax_dim_tensor_contiguous_f32 / _f64 (crates/ft-kernel-cpu/src/lib.rs:39298-39375,
// 18504-18590), cross_entropy_forward_f32 / _f64 (:6717-6738, 6649-6671) and
// cross_entropy_backward_f32 / _f64 (:6745-6781, 6679-6712).
//
// All three are HBM-bound row passes over [rows, classes] logits whose rows (50 257 floats for the
// GPT-2 vocabulary) are neither a vector multiple nor aligned, so a workgroup owns one row and
// moves it with coalesced dword accesses. Rows of up to 65 536 floats (32 768 doubles) are held in
// registers across the max, sum and output steps (64, 256 or 1024 lanes by row length): the row is
// read from HBM once and written once. Longer rows take the streaming kernels, which sweep the row
// three times. Reductions are a fixed per-lane order, a fixed butterfly per wavefront and a fixed
// fold across the wavefronts (the reference scans a row sequentially; same values re-associated,
// inside the parity tolerance), so results are bitwise repeatable. Class indices arrive as int64; an index outside
// [0, classes) (the reference would panic on the slice index) is reported through `bad_index` as
// the lowest offending row, and that row's outputs are left unwritten.

#include <cstdlib>
#include <type_traits>

#include "common.hpp"
#include "devmath.hpp"

namespace {

constexpr int kWave = 64;
constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;

template <typename T> __device__ __forceinline__ T t_exp(T v);
template <> __device__ __forceinline__ float t_exp<float>(float v) { return fth::exp_hw(v); }
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

template <typename T, class F, int WAVES = kWaves> __device__ __forceinline__ T block_reduce(T v, F f, T *red, int &phase) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = f(v, __shfl_xor(v, off, kWave));
    if (WAVES == 1) return v;
    T *buf = red + phase * WAVES;  // alternate halves: one barrier per reduction is enough
    phase ^= 1;
    if (lane == 0) buf[wave] = v;
    __syncthreads();
    T s = buf[0];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) s = f(s, buf[w]);
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

// ---- bounds-checked row accesses ----
// A buffer resource over [base, base + bytes): the hardware returns 0 for a load and drops a store whose byte offset is
// not below `bytes`, so the ragged end of a row needs no per-lane predicate, and the resource lives in scalar registers:
// the only vector register an access needs is the lane's byte offset, shared by every step of the row.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t span_of(const void *base, int bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes < 0 ? 0 : bytes, 0x00020000);
}
typedef unsigned int raw_u2 __attribute__((ext_vector_type(2)));
// non-temporal: rows are read once and outputs never re-read
template <typename T> __device__ __forceinline__ T span_load(__amdgpu_buffer_rsrc_t r, int byte_off);
template <> __device__ __forceinline__ float span_load<float>(__amdgpu_buffer_rsrc_t r, int byte_off) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, byte_off, 0, 2));
}
template <> __device__ __forceinline__ double span_load<double>(__amdgpu_buffer_rsrc_t r, int byte_off) {
    return __builtin_bit_cast(double, __builtin_amdgcn_raw_buffer_load_b64(r, byte_off, 0, 2));
}
__device__ __forceinline__ void span_store(float v, __amdgpu_buffer_rsrc_t r, int byte_off) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned int, v), r, byte_off, 0, 2);
}
__device__ __forceinline__ void span_store(double v, __amdgpu_buffer_rsrc_t r, int byte_off) {
    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(raw_u2, v), r, byte_off, 0, 2);
}
// max that returns the other operand for a NaN (one instruction; of +0 and -0 it returns +0)
__device__ __forceinline__ float max_skip_nan(float a, float b) { return __builtin_fmaxf(a, b); }
__device__ __forceinline__ double max_skip_nan(double a, double b) { return __builtin_fmax(a, b); }

struct MaxSkipNanOp {
    template <typename T> __device__ __forceinline__ T operator()(T a, T b) const { return max_skip_nan(a, b); }
};

// One row per workgroup, held in registers: lane t owns elements t, t + THREADS, ... (VPT of them).
// MODE 0: log-softmax; 1: cross-entropy loss; 2: cross-entropy dlogits; 3: softmax. The maximum of all skips NaN elements
// (f32::max in the reference's log-softmax fold, a strict `>` scan in its cross-entropy: the same value, up to the
// sign of a zero maximum, which none of the outputs depends on beyond the sign of a zero).
enum { kLogSoftmax = 0, kLossForward = 1, kLossBackward = 2, kSoftmax = 3 };

// `lds_steps` further steps of the row (after the VPT register steps) live in dynamic LDS, filled by direct-to-LDS
// loads: with 19 steps (76 KiB) there and at most 64 registers per lane, two 1024-lane workgroups share a compute unit
// and one's loads overlap the other's arithmetic and stores. Each lane reads back only the LDS words its own loads
// wrote, so a wait for the loads is enough and no barrier is needed. MINW: minimum wavefronts per SIMD (sets the
// register budget). FULL: the caller guarantees cols >= VPT * THREADS, so every register step is fully occupied
// (apart from the alignment lead of step 0) and needs no padding.
//
// The kernel is as much bound by vector instructions as by memory (at [8192, 50257] the vector units were busy 60 % of
// the time with the library exponential and per-element predicates), so each pass is kept to the arithmetic proper:
// the step's address and bound are scalar work, padding is applied only where a step can be ragged, and the
// cross-entropy gradient keeps exp(x - max) from the sum pass instead of taking a second exponential.
template <typename T, int VPT, int THREADS, int MODE, int MINW, bool FULL>
__global__ __launch_bounds__(THREADS, MINW) void resident_rows_kernel(const T *__restrict__ x, const int64_t *__restrict__ target,
                                                                     const T *__restrict__ dloss, int64_t cols, T *__restrict__ out,
                                                                     int64_t *bad_index, int lds_steps) {
    constexpr int WAVES = THREADS / kWave;
    constexpr int kElt = (int)sizeof(T);
    // Left free, the scheduler overlaps the exponentials of many elements and spills the row once the register budget
    // is nearly all row data; there the per-element steps are kept in program order instead.
    constexpr bool kPinOrder = THREADS == 1024 && VPT * (int)sizeof(T) * MINW > 384;
    __shared__ T red[2 * WAVES];
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    T *lrow = reinterpret_cast<T *>(lds_raw) + threadIdx.x;  // this lane's word of LDS step 0
    int phase = 0;
    const int64_t i = blockIdx.x;
    int64_t t = 0;
    if (MODE == kLossForward || MODE == kLossBackward) {
        t = target[i];
        if (t < 0 || t >= cols) {  // uniform over the workgroup
            note_bad(bad_index, i);
            return;
        }
    }
    const int tid = threadIdx.x;
    // Lane slots are counted from the last 64-element boundary at or before the row's first output element (first
    // input element for the loss, which writes no row), so every wavefront store covers whole, aligned 256-byte
    // (fp64: 512-byte) pieces: rows of an odd length start at arbitrary element offsets, and partial-line
    // writes from different wavefronts cost far more HBM time than they carry. Slot j holds element j - lead;
    // slots below `lead` (only in step 0) and from `n` on are empty.
    const T *row_in = x + i * cols;
    const T *row_out = (MODE == kLossForward ? x : out) + i * cols;
    const int lead = (int)((reinterpret_cast<uintptr_t>(row_out) / sizeof(T)) % kWave);
    const T *xr = row_in - lead;         // slot 0 of the row
    const int n = (int)cols + lead;      // one past the last occupied slot
    const int kfull = n / THREADS;       // steps below this one are full, step kfull is ragged, later ones are empty
    // LDS steps [0, lds_full) are full; the (at most two) remaining ones take a per-lane bound
    const int lds_full = kfull - VPT < 0 ? 0 : (kfull - VPT < lds_steps ? kfull - VPT : lds_steps);
    if constexpr (sizeof(T) == 4) {
        // oldest in the load queue, so the compiler's own counted waits for the register loads below stay exact
        const unsigned wave = __builtin_amdgcn_readfirstlane((unsigned)(tid / kWave));
        const unsigned wave_base = __builtin_amdgcn_readfirstlane((unsigned)reinterpret_cast<uintptr_t>(lds_raw)) + wave * (kWave * 4u);
        const unsigned lane_off = (unsigned)(tid & (kWave - 1)) * 4u;
        for (int k = 0; k < lds_steps; ++k) {
            const T *pk = xr + (VPT + k) * THREADS + wave * kWave;  // scalar: the wavefront's 64 slots of step VPT + k
            if (k < lds_full || tid < n - (VPT + k) * THREADS)
                asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1 nt" ::"v"(lane_off), "s"(pk),
                             "s"(wave_base + (unsigned)k * (THREADS * 4u))
                             : "memory", "m0");
        }
    }
    // Step k touches slots [k * THREADS, (k + 1) * THREADS) through a resource that starts at the step's slot 0 and ends
    // with the row: scalar work per step, and the one per-lane offset `off` for all of them.
    const int off = tid * kElt;
    const bool lead_ok = tid >= lead;
    auto step_span = [&](const T *slot0, int k, int end) __attribute__((always_inline)) {
        return span_of(slot0 + k * THREADS, (end - k * THREADS) * kElt);
    };
    T v[VPT];
    {
        // step 0: the `lead` empty slots lie before the row (for row 0, before the allocation): their lanes read
        // element 0 and drop it
        const int e0 = tid - lead;
        const T t0 = span_load<T>(span_of(row_in, (int)cols * kElt), (e0 < 0 ? 0 : e0) * kElt);
        v[0] = (lead_ok && tid < n) ? t0 : T(-__builtin_inf());
    }
#pragma unroll
    for (int k = 1; k < VPT; ++k) {
        const T tk = span_load<T>(step_span(xr, k, n), off);
        v[k] = (FULL || tid < n - k * THREADS) ? tk : T(-__builtin_inf());
    }
    T m = T(-__builtin_inf());
#pragma unroll
    for (int k = 0; k < VPT; ++k) m = max_skip_nan(m, v[k]);  // the padding never wins
    if (lds_steps > 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    for (int k = 0; k < lds_full; ++k) m = max_skip_nan(m, lrow[k * THREADS]);
    for (int k = lds_full; k < lds_steps; ++k)
        if (tid < n - (VPT + k) * THREADS) m = max_skip_nan(m, lrow[k * THREADS]);
    m = block_reduce<T, MaxSkipNanOp, WAVES>(m, MaxSkipNanOp{}, red, phase);
    // The -inf padding adds exp(-inf - m) = +0 for a finite or +inf maximum and NaN for a -inf one, where the sum of
    // the real elements is NaN already, so the sum over the registers needs no bounds test. The gradient keeps
    // e = exp(x - m) in place of x: its output is e / sum.
    T s = T(0);
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const T e = t_exp<T>(v[k] - m);
        s += e;
        if (MODE == kLossBackward || MODE == kSoftmax) v[k] = e;
        if (kPinOrder) __builtin_amdgcn_sched_barrier(0);
    }
    auto lds_sum = [&](int k) __attribute__((always_inline)) {
        const T e = t_exp<T>(lrow[k * THREADS] - m);
        s += e;
        if (MODE == kLossBackward || MODE == kSoftmax) lrow[k * THREADS] = e;
    };
    for (int k = 0; k < lds_full; ++k) lds_sum(k);
    for (int k = lds_full; k < lds_steps; ++k)
        if (tid < n - (VPT + k) * THREADS) lds_sum(k);
    s = block_reduce<T, SumOp, WAVES>(s, SumOp{}, red, phase);
    if (MODE == kLossForward) {
        if (tid == 0) out[i] = (m + t_log<T>(s)) - x[i * cols + t];
        return;
    }
    // Outputs: step 0 is stored under the lane's own predicate (an offset before the row must not reach memory), every
    // other step through its bounded resource. Values computed from empty slots are dropped by the bound.
    T *yr = out + i * cols - lead;
    // The bounds of the output steps equal those of the input steps; recomputing them from an opaque copy of `n` costs one
    // scalar instruction per step, where keeping 32 of them alive across the kernel spills scalar registers.
    int n_out = n;
    asm volatile("" : "+s"(n_out));
    const T lse = t_log<T>(s);                                     // log-softmax: (x - m) - ln(sum)
    const T inv_s = T(1) / s, g = MODE == kLossBackward ? dloss[i] : T(0);  // gradient: g (e / sum - onehot)
    const int tt = (int)t + lead;                                  // the target's slot
    auto result = [&](T val, int slot0_of_step) __attribute__((always_inline)) {
        if (MODE == kLogSoftmax) return (val - m) - lse;
        if (MODE == kSoftmax) return val * inv_s;  // one correctly rounded 1 / sum per row, as the 128-bit row kernel
        return g * (val * inv_s - (tid == tt - slot0_of_step ? T(1) : T(0)));
    };
    if (lead_ok) span_store(result(v[0], 0), span_of(out + i * cols, (int)cols * kElt), (tid - lead) * kElt);
#pragma unroll
    for (int k = 1; k < VPT; ++k) {
        span_store(result(v[k], k * THREADS), step_span(yr, k, n_out), off);
        if (kPinOrder) __builtin_amdgcn_sched_barrier(0);
    }
    for (int k = 0; k < lds_steps; ++k) span_store(result(lrow[k * THREADS], (VPT + k) * THREADS), step_span(yr, VPT + k, n_out), off);
}

// Cross-entropy loss of long fp32 rows in one streaming pass. The loss needs only the row's log-sum-exp and one
// element, so nothing of the row has to stay on chip: each lane keeps a running maximum m and the sum s of exp(v - m) over
// the elements it has seen, rescaling s when a batch of 32 values raises m (one extra exponential per batch at most), and
// the lanes' pairs are merged at the end. Against the two-pass form (maximum first, then the sum) only the rounding of s
// differs, by a few ulp. The row is read as a scalar head up to the first 16-byte boundary, 128-bit non-temporal vectors
// eight deep per lane, and a scalar tail (rows such as 50 257 floats start at arbitrary 4-byte offsets). m starts at the
// lowest finite value, not -inf: a -inf element then adds exp(-inf) = 0 instead of exp(-inf + inf), as it does in the
// two-pass form whenever the row holds one finite value; a row of nothing but -inf ends as m + ln 0 - (-inf) = NaN, as
// there. NaN elements never raise m (strict >) and poison s, +inf gives exp(inf - inf): NaN, as there.
__global__ __launch_bounds__(256) void cross_entropy_forward_stream_kernel(const float *__restrict__ logits, const int64_t *__restrict__ target,
                                                                           int64_t classes, float *__restrict__ loss, int64_t *bad_index) {
    constexpr int NT = 256, WAVES = NT / kWave;
    typedef float nat_f4 __attribute__((ext_vector_type(4)));
    __shared__ float red[2 * WAVES];
    int phase = 0;
    const int64_t i = blockIdx.x;
    const int64_t t = target[i];
    if (t < 0 || t >= classes) {  // uniform over the workgroup
        note_bad(bad_index, i);
        return;
    }
    const float *xr = logits + i * classes;
    float m = -3.402823466e+38f, s = 0.f;
    auto feed1 = [&](float v) __attribute__((always_inline)) {
        const float nm = max_gt(m, v);
        if (nm > m) {
            s *= t_exp<float>(m - nm);
            m = nm;
        }
        s += t_exp<float>(v - m);
    };
    int64_t lead = (int64_t)(((16u - (unsigned)(reinterpret_cast<uintptr_t>(xr) & 15u)) & 15u) / sizeof(float));
    if (lead > classes) lead = classes;
    if ((int64_t)threadIdx.x < lead) feed1(xr[threadIdx.x]);
    const int64_t nvec = (classes - lead) / 4;
    const nat_f4 *xv = reinterpret_cast<const nat_f4 *>(xr + lead);
    int64_t j = threadIdx.x;
    // The body of the row: 32 values per lane and trip. Only the SUM of the exponentials is needed, so they are taken as a bare
    // 2^((v - m) log2 e) on the hardware unit (three instructions; relative error |v - m| 2^-24 per term, i.e. below 1e-6 for every
    // term that is not negligible, and the terms that carry the sum have small |v - m|) and the maximum as v_max3 (which skips
    // NaN exactly as the strict `>` scan does): 4.5 vector instructions per element where the compensated exponential and the
    // compare-and-select maximum took 13 -- this kernel's vector units were busy 0.60 of its cycles. Four partial sums per lane
    // (one per vector component) keep the adds from forming one dependent chain.
    constexpr float kLog2e = 1.44269502162933349609375f;
    float s4[4] = {0.f, 0.f, 0.f, 0.f};
    for (; j + 7 * NT < nvec; j += 8 * NT) {
        nat_f4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(xv + j + u * NT);
        float nm = m;
#pragma unroll
        for (int u = 0; u < 8; ++u) nm = __builtin_fmaxf(nm, __builtin_fmaxf(__builtin_fmaxf(v[u].x, v[u].y), __builtin_fmaxf(v[u].z, v[u].w)));
        if (nm > m) {
            const float f = t_exp<float>(m - nm);
            s *= f;
#pragma unroll
            for (int c = 0; c < 4; ++c) s4[c] *= f;
            m = nm;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            s4[0] += __builtin_amdgcn_exp2f((v[u].x - m) * kLog2e);
            s4[1] += __builtin_amdgcn_exp2f((v[u].y - m) * kLog2e);
            s4[2] += __builtin_amdgcn_exp2f((v[u].z - m) * kLog2e);
            s4[3] += __builtin_amdgcn_exp2f((v[u].w - m) * kLog2e);
        }
    }
    s += (s4[0] + s4[1]) + (s4[2] + s4[3]);
    for (; j < nvec; j += NT) {
        const nat_f4 v = __builtin_nontemporal_load(xv + j);
        feed1(v.x);
        feed1(v.y);
        feed1(v.z);
        feed1(v.w);
    }
    const int64_t t0 = lead + nvec * 4 + threadIdx.x;
    if (t0 < classes) feed1(xr[t0]);
    const float m_all = block_reduce<float, MaxGtOp, WAVES>(m, MaxGtOp{}, red, phase);
    const float s_all = block_reduce<float, SumOp, WAVES>(s * t_exp<float>(m - m_all), SumOp{}, red, phase);
    if (threadIdx.x == 0) loss[i] = (m_all + t_log<float>(s_all)) - xr[t];
}

// Launches the register-resident kernel if the row fits; returns false if it does not (the caller streams).
template <typename T, int MODE>
bool launch_resident(const T *x, const int64_t *target, const T *dloss, int64_t rows, int64_t cols, T *out, int64_t *bad_index,
                     hipStream_t st) {
    constexpr int kMaxVpt = sizeof(T) == 4 ? 64 : 32;
    const int64_t slots = cols + (kWave - 1);  // the row plus the longest alignment lead
    if (slots > 1024LL * kMaxVpt) return false;
    const int64_t steps = fth::ceil_div(slots, (int64_t)1024);
    if constexpr (sizeof(T) == 4) {
        // fp32 rows of 25..51 steps of 1024: up to 19 steps in LDS, the rest (8..32 steps) in registers, two workgroups
        // per compute unit. Longer rows keep the whole row in registers at one workgroup per compute unit.
        constexpr int64_t kLdsSteps = 19;
        if (steps > 24 && steps <= 32 + kLdsSteps) {
            const int64_t need = steps - kLdsSteps;
#define FTH_HYBRID(VPT)                                                                                                         \
    if (need <= (VPT)) {                                                                                                       \
        const int lds_steps = (int)(steps - (VPT));                                                                            \
        resident_rows_kernel<T, VPT, 1024, MODE, 8, true><<<dim3((unsigned)rows), dim3(1024), (size_t)lds_steps * 4096, st>>>(       \
            x, target, dloss, cols, out, bad_index, lds_steps);                                                                \
        return true;                                                                                                           \
    }
            FTH_HYBRID(8)
            FTH_HYBRID(16)
            FTH_HYBRID(24)
            FTH_HYBRID(32)
#undef FTH_HYBRID
        }
    }
#define FTH_RESIDENT(THREADS, VPT)                                                                                                  \
    if (slots <= (int64_t)(THREADS) * (VPT)) {                                                                                     \
        if constexpr ((VPT) <= kMaxVpt)                                                                                            \
            resident_rows_kernel<T, VPT, THREADS, MODE, 1, false><<<dim3((unsigned)rows), dim3(THREADS), 0, st>>>(x, target, dloss, cols, \
                                                                                                            out, bad_index, 0);    \
        return true;                                                                                                               \
    }
    FTH_RESIDENT(64, 4)
    FTH_RESIDENT(64, 16)
    FTH_RESIDENT(256, 8)
    FTH_RESIDENT(256, 16)
    FTH_RESIDENT(256, 32)
    FTH_RESIDENT(1024, 16)
    FTH_RESIDENT(1024, 24)
    FTH_RESIDENT(1024, 32)
    FTH_RESIDENT(1024, 40)
    FTH_RESIDENT(1024, 48)
    FTH_RESIDENT(1024, 56)
    FTH_RESIDENT(1024, 64)
#undef FTH_RESIDENT
    return false;
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
        if (!launch_resident<T, kLogSoftmax>(x, nullptr, nullptr, outer, reduce, y, nullptr, st))
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
        if (backward) {
            if (!launch_resident<T, kLossBackward>(logits, target, dloss, batch, classes, out, bad_index, st))
                cross_entropy_backward_kernel<T><<<dim3((unsigned)batch), dim3(kThreads), 0, st>>>(logits, target, dloss, classes, out, bad_index);
        } else {
            bool streamed = false;
            if constexpr (std::is_same<T, float>::value) {
                static const bool stream_off = [] {
                    const char *e = std::getenv("FT_HIP_CE_STREAM");  // tuning knob: 0 keeps the row-resident loss kernel for long rows
                    return e && std::atoi(e) == 0;
                }();
                if (!stream_off && classes >= 8192) {  // long rows: one streaming pass, nothing of the row kept on chip
                    // (three workgroups per compute unit read the stream fastest, as for the argmax kernel: 48 KiB of unused dynamic LDS
                    //  per workgroup hold the count there, whatever the register allocation would allow)
                    cross_entropy_forward_stream_kernel<<<dim3((unsigned)batch), dim3(256), (size_t)48 * 1024, st>>>(logits, target, classes, out,
                                                                                                                    bad_index);
                    streamed = true;
                }
            }
            if (!streamed && !launch_resident<T, kLossForward>(logits, target, nullptr, batch, classes, out, bad_index, st))
                cross_entropy_forward_kernel<T><<<dim3((unsigned)batch), dim3(kThreads), 0, st>>>(logits, target, classes, out, bad_index);
        }
        FTH_CHECK_LAUNCH("cross_entropy");
    }
    if (bad_index) {
        finish_bad_index_kernel<<<1, 1, 0, st>>>(bad_index);
        FTH_CHECK_LAUNCH("cross_entropy_bad_index");
    }
    return FTH_OK;
}

}  // namespace

namespace fth {
bool softmax_resident_rows(const float *x, float *y, int64_t rows, int64_t cols, hipStream_t st) {
    return launch_resident<float, kSoftmax>(x, nullptr, nullptr, rows, cols, y, nullptr, st);
}
bool softmax_resident_rows(const double *x, double *y, int64_t rows, int64_t cols, hipStream_t st) {
    return launch_resident<double, kSoftmax>(x, nullptr, nullptr, rows, cols, y, nullptr, st);
}
}  // namespace fth

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
