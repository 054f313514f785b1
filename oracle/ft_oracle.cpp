// TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// CPU restatement of the transformer forward ops of the reference's `ft-kernel-cpu` crate, used
// only as the checker in tests/, in __graft_entry__.smoke() and as the `cpu_baseline` leg of
// bench.py. Nothing under frankentorch_amd/ links, loads or calls this file.
//
// Build: g++ -O2 -ffp-contract=off -fno-fast-math -fopenmp (see oracle/build_oracle.py). The
// reference is Rust, which never contracts a*b+c into an FMA, hence -ffp-contract=off.
//
// Each function cites the reference lines it follows (paths relative to the reference root;
// KC = crates/ft-kernel-cpu/src/lib.rs). Parity status per function:
//   pinned by the reference's own fixtures / closed forms (tests/test_oracle_golden.py):
//     softmax, gelu, add, matmul (small exact + stored f64 checksums), bmm, addmm, linear,
//     index_select, argmax, layer_norm / rms_norm (closed form + textbook), sdpa (textbook
//     attention + brute force), permute;
//     layer_norm / rms_norm / linear / sdpa backward: central differences of the pinned forward
//     functions in f64, the reference's own test inputs (KC:43862-43911, 64200-64360) and the
//     identities those tests assert (unit-dy shortcut, dbias = column sums);
//     log_softmax: the reference's conformance fixtures (1e-10) and log(softmax); cross-entropy forward /
//     backward: -log_softmax[target], central differences, rows of the gradient summing to zero.
//     masked / grouped-query sdpa: the reference's expand-then-masked identity on its own inputs (KC:45159-45218), an einsum
//     restatement, reduction to the pinned unmasked and causal forms; masked sdpa backward (KC:5423): central differences of
//     the pinned masked forward, the same reductions, an einsum restatement; unit-dOut sdpa backward (KC:5662): the
//     reference's own test against dense ones on its inputs and bound (KC:45119-45155);
//     tanh gelu: ft-nn's golden values and torch's CPU kernel; int8 quantisers and linear: the reference's tie vector and
//     scale (KC:43721-43740), its accuracy bounds on its LCG inputs (KC:43645-43708), an independent integer product.
//   parity unpinned: none of the functions in this file (what the checkout cannot pin -- session RNG dependent golden files,
//     kernel routing inside the missing ft-api crate, matrixmultiply's bit digests -- is not restated here).
//   third-party arithmetic that is NOT in the reference tree:
//     * GEMM: `matrixmultiply 0.3.11` (Cargo.lock:1420-1423; call sites KC:1645, KC:1673). Its
//       f32 accumulation order is unspecified and the reference's own test shows it is not the
//       sequential-k sum (KC:50617-50689). fto_gemm_f32 therefore accumulates in f64 and rounds
//       once: the exact product to within 2^-24 relative, which every order matrixmultiply
//       could use must also approach. Tolerance parity only; bit parity with matrixmultiply is
//       unreachable and not claimed.
//     * erff / erf: `libm 0.2.16` (Cargo.lock:1366-1369; KC:36968, KC:1928), a port of
//       FreeBSD msun. This file calls the platform libm (glibc) instead; both are documented
//       <= 1 ULP, and the reference's gelu fixture (5 points, 1e-10) pins the f64 form.
//     * expf / exp: Rust std calls the platform libm, as this file does.

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

#if defined(__x86_64__)
#include <immintrin.h>
#endif

extern "C" {

// ------------------------------------------------------------------------------------------
// Threads (the reference's rayon pool defaults to one worker per logical core,
// crates/ft-kernel-cpu/src/pool.rs:5-8; size gates never change results, KC:2576, 3053, 5773)
// ------------------------------------------------------------------------------------------
int fto_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
void fto_set_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

}  // extern "C"

namespace {

// pairwise_sum_f32 / _f64 (KC:37521-37528): <= 128 elements sequentially, else split at len / 2.
template <typename T> T pairwise_sum(const T *v, size_t n) {
    if (n <= 128) {
        T s = 0;
        for (size_t i = 0; i < n; ++i) s += v[i];
        return s;
    }
    size_t mid = n / 2;
    return pairwise_sum(v, mid) + pairwise_sum(v + mid, n - mid);
}

// f32::max / f64::max (IEEE maxNum: a NaN operand is ignored), as used in the fold at KC:39221.
template <typename T> T max_num(T a, T b) {
    if (a != a) return b;
    if (b != b) return a;
    return a > b ? a : b;
}

inline float t_exp(float x) { return expf(x); }
inline double t_exp(double x) { return exp(x); }
inline float t_erf(float x) { return erff(x); }
inline double t_erf(double x) { return erf(x); }
inline float t_sqrt(float x) { return sqrtf(x); }
inline double t_sqrt(double x) { return sqrt(x); }

// softmax_dim_tensor_contiguous_f32 (KC:39193-39296), _f64 (KC:18350-18461): per lane,
// max = fold(-inf, max); out = exp(x - max); sum = pairwise_sum(out); out /= sum.
template <typename T> void softmax_impl(const T *x, T *y, int64_t outer, int64_t reduce, int64_t inner) {
    if (outer <= 0 || reduce <= 0 || inner <= 0) return;
    if (inner == 1) {
#pragma omp parallel for schedule(static)
        for (int64_t o = 0; o < outer; ++o) {
            const T *in = x + o * reduce;
            T *out = y + o * reduce;
            T m = -std::numeric_limits<T>::infinity();
            for (int64_t j = 0; j < reduce; ++j) m = max_num(m, in[j]);
            for (int64_t j = 0; j < reduce; ++j) out[j] = t_exp(in[j] - m);
            T s = pairwise_sum(out, (size_t)reduce);
            for (int64_t j = 0; j < reduce; ++j) out[j] /= s;
        }
        return;
    }
#pragma omp parallel
    {
        std::vector<T> scratch((size_t)reduce);
#pragma omp for schedule(static)
        for (int64_t o = 0; o < outer; ++o) {
            const T *in = x + o * reduce * inner;
            T *out = y + o * reduce * inner;
            for (int64_t c = 0; c < inner; ++c) {
                for (int64_t r = 0; r < reduce; ++r) scratch[r] = in[r * inner + c];
                T m = -std::numeric_limits<T>::infinity();
                for (int64_t r = 0; r < reduce; ++r) m = max_num(m, scratch[r]);
                for (int64_t r = 0; r < reduce; ++r) scratch[r] = t_exp(scratch[r] - m);
                T s = pairwise_sum(scratch.data(), (size_t)reduce);
                for (int64_t r = 0; r < reduce; ++r) out[r * inner + c] = scratch[r] / s;
            }
        }
    }
}

// layer_norm_forward_f32 (KC:5877-5923), _f64 (KC:5824-5870); with `b2` non-null it is
// add_layer_norm_forward_f32 (KC:5932-5984): a + b materialised once, then the same passes.
template <typename T>
void layer_norm_impl(const T *x, const T *x2, const T *w, const T *b, T *y, int64_t batch, int64_t n, T eps) {
    if (batch <= 0 || n <= 0) return;
    const T inv_n = T(1) / (T)n;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < batch; ++r) {
        const T *xr = x + r * n;
        T *o = y + r * n;
        T sum = 0;
        if (x2) {
            const T *x2r = x2 + r * n;
            for (int64_t j = 0; j < n; ++j) {
                T s = xr[j] + x2r[j];
                o[j] = s;
                sum += s;
            }
            xr = o;
        } else {
            for (int64_t j = 0; j < n; ++j) sum += xr[j];
        }
        const T mean = sum * inv_n;
        T vsum = 0;
        for (int64_t j = 0; j < n; ++j) {
            T d = xr[j] - mean;
            vsum += d * d;
        }
        const T rstd = T(1) / t_sqrt(vsum * inv_n + eps);
        for (int64_t j = 0; j < n; ++j) {
            T v = (xr[j] - mean) * rstd;
            if (w) v *= w[j];
            if (b) v += b[j];
            o[j] = v;
        }
    }
}

// rms_norm_forward_f32 (KC:6459-6494), _f64 (KC:6418-6453).
template <typename T> void rms_norm_impl(const T *x, const T *w, T *y, int64_t batch, int64_t n, T eps) {
    if (batch <= 0 || n <= 0) return;
    const T inv_n = T(1) / (T)n;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < batch; ++r) {
        const T *xr = x + r * n;
        T *o = y + r * n;
        T ss = 0;
        for (int64_t j = 0; j < n; ++j) ss += xr[j] * xr[j];
        const T rstd = T(1) / t_sqrt(ss * inv_n + eps);
        for (int64_t j = 0; j < n; ++j) {
            T v = xr[j] * rstd;
            if (w) v *= w[j];
            o[j] = v;
        }
    }
}

// gelu_value_f32 (KC:36966-36969); f64 form KC:1924-1929.
inline float gelu_value(float x) { return 0.5f * x * (1.0f + t_erf(x * 0.70710678118654752440f)); }
inline double gelu_value(double x) { return 0.5 * x * (1.0 + t_erf(x * 0.70710678118654752440)); }
// tanh-form GELU: the `gelu` kernel of the fused GPU module (crates/ft-kernel-metal/src/fused.rs:301-313, f32, with its
// |x| >= 10 clamp; the CPU check of that kernel at :1256-1259 uses the same expression) and GELU::tanh()
// (crates/ft-nn/src/lib.rs:1924-1957; four golden values at :21985-22004).
inline float gelu_tanh_value(float x) {
    if (x >= 10.0f) return x;
    if (x <= -10.0f) return 0.0f;
    return 0.5f * x * (1.0f + std::tanh(0.7978845608028654f * (x + 0.044715f * x * x * x)));
}
inline double gelu_tanh_value(double x) { return 0.5 * x * (1.0 + std::tanh(0.79788456080286535588 * (x + 0.044715 * x * x * x))); }

// GEMM truth for f32: accumulate in f64 (each product of two f32 is exact in f64), round once.
// b_kn is [k, n] row-major with pitch ldb.
void gemm_f32_kn(int64_t m, int64_t n, int64_t k, const float *a, int64_t lda, const float *b, int64_t ldb,
                 float *c, int64_t ldc) {
#pragma omp parallel
    {
        std::vector<double> acc((size_t)n);
#pragma omp for schedule(dynamic, 4)
        for (int64_t i = 0; i < m; ++i) {
            std::fill(acc.begin(), acc.end(), 0.0);
            const float *ar = a + i * lda;
            for (int64_t p = 0; p < k; ++p) {
                const double av = (double)ar[p];
                const float *br = b + p * ldb;
                double *ac = acc.data();
                for (int64_t j = 0; j < n; ++j) ac[j] += av * (double)br[j];
            }
            float *cr = c + i * ldc;
            for (int64_t j = 0; j < n; ++j) cr[j] = (float)acc[j];
        }
    }
}

// GEMM truth for f64: accumulate in long double (x87 80-bit), round once.
void gemm_f64_kn(int64_t m, int64_t n, int64_t k, const double *a, int64_t lda, const double *b, int64_t ldb,
                 double *c, int64_t ldc) {
#pragma omp parallel
    {
        std::vector<long double> acc((size_t)n);
#pragma omp for schedule(dynamic, 4)
        for (int64_t i = 0; i < m; ++i) {
            std::fill(acc.begin(), acc.end(), 0.0L);
            const double *ar = a + i * lda;
            for (int64_t p = 0; p < k; ++p) {
                const long double av = (long double)ar[p];
                const double *br = b + p * ldb;
                for (int64_t j = 0; j < n; ++j) acc[j] += av * (long double)br[j];
            }
            double *cr = c + i * ldc;
            for (int64_t j = 0; j < n; ++j) cr[j] = (double)acc[j];
        }
    }
}

template <typename T> void transpose_nk_to_kn(const T *w, int64_t n, int64_t k, int64_t ldw, std::vector<T> &out) {
    out.resize((size_t)n * (size_t)k);
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < n; ++j)
        for (int64_t p = 0; p < k; ++p) out[(size_t)p * n + j] = w[j * ldw + p];
}

void gemm_any(int trans_b, int64_t m, int64_t n, int64_t k, const float *a, int64_t lda, const float *b, int64_t ldb,
              float *c, int64_t ldc) {
    if (m <= 0 || n <= 0) return;
    if (!trans_b) return gemm_f32_kn(m, n, k, a, lda, b, ldb, c, ldc);
    std::vector<float> t;
    transpose_nk_to_kn(b, n, k, ldb, t);
    gemm_f32_kn(m, n, k, a, lda, t.data(), n, c, ldc);
}
void gemm_any(int trans_b, int64_t m, int64_t n, int64_t k, const double *a, int64_t lda, const double *b,
              int64_t ldb, double *c, int64_t ldc) {
    if (m <= 0 || n <= 0) return;
    if (!trans_b) return gemm_f64_kn(m, n, k, a, lda, b, ldb, c, ldc);
    std::vector<double> t;
    transpose_nk_to_kn(b, n, k, ldb, t);
    gemm_f64_kn(m, n, k, a, lda, t.data(), n, c, ldc);
}

// linear_tensor_f32 (KC:17306-17353): y = x . W^T, then the bias pass on the rounded result.
template <typename T>
void linear_impl(const T *x, const T *w, const T *bias, int64_t batch, int64_t in_f, int64_t out_f, T *y) {
    if (batch <= 0 || out_f <= 0) return;
    gemm_any(1, batch, out_f, in_f, x, in_f, w, in_f, y, out_f);
    if (bias) {
#pragma omp parallel for schedule(static)
        for (int64_t r = 0; r < batch; ++r)
            for (int64_t j = 0; j < out_f; ++j) y[r * out_f + j] += bias[j];
    }
}

// sdpa_forward_f32 (KC:5200-5284), _f64 (KC:4572-4651). The block height cannot change results
// (KC:4982-4984), so rows are processed one at a time. The two GEMMs are the f64-accumulated
// truth; the row softmax between them is the reference's scalar loop verbatim (KC:5238-5256):
// scale after the product, strict `>` max scan over the first `limit` entries, exp, sequential
// sum, divide, zero the tail.
template <typename T>
void sdpa_impl(const T *q, const T *k, const T *v, int64_t num_bh, int64_t seq_q, int64_t seq_k, int64_t d_k,
               int64_t d_v, T scale, int causal, T *out) {
    if (num_bh <= 0 || seq_q <= 0 || d_v <= 0) return;
    using Wide = typename std::conditional<sizeof(T) == 4, double, long double>::type;
#pragma omp parallel
    {
        std::vector<T> sc((size_t)std::max<int64_t>(seq_k, 1));
        std::vector<Wide> acc((size_t)d_v);
#pragma omp for schedule(dynamic, 8) collapse(2)
        for (int64_t bh = 0; bh < num_bh; ++bh) {
            for (int64_t qi = 0; qi < seq_q; ++qi) {
                const T *qr = q + (bh * seq_q + qi) * d_k;
                const T *kh = k + bh * seq_k * d_k;
                const T *vh = v + bh * seq_k * d_v;
                // gemm::sgemm_bt(br, d_k, seq_k, q_block, kh, sc): the FULL row of scores, KC:5229
                for (int64_t j = 0; j < seq_k; ++j) {
                    Wide dot = 0;
                    const T *kr = kh + j * d_k;
                    for (int64_t c = 0; c < d_k; ++c) dot += (Wide)qr[c] * (Wide)kr[c];
                    sc[j] = (T)dot;
                }
                const int64_t limit = causal ? std::min<int64_t>(qi + 1, seq_k) : seq_k;
                T m = -std::numeric_limits<T>::infinity();
                for (int64_t j = 0; j < limit; ++j) {
                    sc[j] *= scale;
                    if (sc[j] > m) m = sc[j];
                }
                T sum = 0;
                for (int64_t j = 0; j < limit; ++j) {
                    T e = t_exp(sc[j] - m);
                    sc[j] = e;
                    sum += e;
                }
                for (int64_t j = 0; j < limit; ++j) sc[j] /= sum;
                for (int64_t j = limit; j < seq_k; ++j) sc[j] = 0;
                // gemm::sgemm(br, seq_k, d_v, sc, vh, o_block), KC:5258
                std::fill(acc.begin(), acc.end(), (Wide)0);
                for (int64_t j = 0; j < seq_k; ++j) {
                    const Wide pj = (Wide)sc[j];
                    const T *vr = vh + j * d_v;
                    for (int64_t c = 0; c < d_v; ++c) acc[c] += pj * (Wide)vr[c];
                }
                T *o = out + (bh * seq_q + qi) * d_v;
                for (int64_t c = 0; c < d_v; ++c) o[c] = (T)acc[c];
            }
        }
    }
}

// sdpa_forward_masked_gqa_f64 (KC:4777-4850); sdpa_forward_masked_f64 (KC:4661-4741) is the h_q == h_kv case. q is
// [batch, h_q, seq_q, d_k]; k / v are [batch, h_kv, seq_k, d_*]; query head hq reads K/V head hq / (h_q / h_kv).
// scores = (q . k^T) * scale + mask over ALL seq_k keys (the additive mask carries any causality as -inf); max by a
// strict `>` scan; e = exp(s - m); s /= sum; out = p . v. mask_bh_stride is 0 (one [seq_q, seq_k] mask for every head)
// or seq_q * seq_k (one per batch*h_q). The reference has the f64 form only; the f32 instantiation is the same steps.
template <typename T>
void sdpa_masked_gqa_impl(const T *q, const T *k, const T *v, int64_t batch, int64_t h_q, int64_t h_kv, int64_t seq_q, int64_t seq_k,
                          int64_t d_k, int64_t d_v, T scale, const T *mask, int64_t mask_bh_stride, T *out) {
    const int64_t num_bh = batch * h_q;
    if (num_bh <= 0 || seq_q <= 0 || d_v <= 0 || h_kv <= 0) return;
    const int64_t group = h_q / h_kv;
    using Wide = typename std::conditional<sizeof(T) == 4, double, long double>::type;
#pragma omp parallel
    {
        std::vector<T> sc((size_t)std::max<int64_t>(seq_k, 1));
        std::vector<Wide> acc((size_t)d_v);
#pragma omp for schedule(dynamic, 8) collapse(2)
        for (int64_t bh = 0; bh < num_bh; ++bh) {
            for (int64_t qi = 0; qi < seq_q; ++qi) {
                const int64_t b = bh / h_q, kv_head = (bh % h_q) / group;  // KC:4812-4813
                const T *qr = q + (bh * seq_q + qi) * d_k;
                const T *kh = k + (b * h_kv + kv_head) * seq_k * d_k;
                const T *vh = v + (b * h_kv + kv_head) * seq_k * d_v;
                const T *mrow = mask + bh * mask_bh_stride + qi * seq_k;
                for (int64_t j = 0; j < seq_k; ++j) {  // dgemm_bt, KC:4823
                    Wide dot = 0;
                    const T *kr = kh + j * d_k;
                    for (int64_t c = 0; c < d_k; ++c) dot += (Wide)qr[c] * (Wide)kr[c];
                    sc[j] = (T)dot;
                }
                T m = -std::numeric_limits<T>::infinity();
                for (int64_t j = 0; j < seq_k; ++j) {  // KC:4829-4834
                    sc[j] = sc[j] * scale + mrow[j];
                    if (sc[j] > m) m = sc[j];
                }
                T sum = 0;
                for (int64_t j = 0; j < seq_k; ++j) {
                    T e = t_exp(sc[j] - m);
                    sc[j] = e;
                    sum += e;
                }
                for (int64_t j = 0; j < seq_k; ++j) sc[j] /= sum;
                std::fill(acc.begin(), acc.end(), (Wide)0);
                for (int64_t j = 0; j < seq_k; ++j) {  // dgemm, KC:4846
                    const Wide pj = (Wide)sc[j];
                    const T *vr = vh + j * d_v;
                    for (int64_t c = 0; c < d_v; ++c) acc[c] += pj * (Wide)vr[c];
                }
                T *o = out + (bh * seq_q + qi) * d_v;
                for (int64_t c = 0; c < d_v; ++c) o[c] = (T)acc[c];
            }
        }
    }
}

// quantize_rows_i8 (KC:37879-37905) and quantize_per_output_channel_i8 (KC:37836-37868): per row, amax = fold(0, max(acc, |v|))
// (f32::max ignores a NaN operand), scale = amax > 0 ? amax / 127 : 1, q = clamp(round_ties_even(v / scale), -127, 127) as i8
// (`as i8` turns NaN into 0).
void quantize_rows_i8_impl(const float *x, int64_t rows, int64_t cols, int8_t *q, float *scales) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float *row = x + r * cols;
        float amax = 0.0f;
        for (int64_t i = 0; i < cols; ++i) amax = std::fmax(amax, std::fabs(row[i]));
        const float scale = amax > 0.0f ? amax / 127.0f : 1.0f;
        for (int64_t i = 0; i < cols; ++i) {
            const float v = std::nearbyintf(row[i] / scale);  // default rounding mode: ties to even
            q[r * cols + i] = (v != v) ? (int8_t)0 : (int8_t)std::fmin(std::fmax(v, -127.0f), 127.0f);
        }
        scales[r] = scale;
    }
}

// linear_int8_dynamic_f32 (KC:37966-38060): quantise x per row, i32 dot products (dot_i8, KC:38282-38313), then
// y = acc as f32 * a_scale * w_scale (+ bias), the three float operations in that order.
void linear_int8_dynamic_impl(const float *x, int64_t m, int64_t k, const int8_t *w_i8, const float *w_scales, int64_t n, const float *bias,
                              float *out) {
    std::vector<int8_t> xq((size_t)(m * k));
    std::vector<float> a_scales((size_t)m);
    quantize_rows_i8_impl(x, m, k, xq.data(), a_scales.data());
#pragma omp parallel for schedule(static)
    for (int64_t s = 0; s < m; ++s) {
        const int8_t *xr = xq.data() + s * k;
        for (int64_t o = 0; o < n; ++o) {
            const int8_t *wr = w_i8 + o * k;
            int32_t acc = 0;
            for (int64_t i = 0; i < k; ++i) acc += (int32_t)xr[i] * (int32_t)wr[i];
            float y = (float)acc * a_scales[s] * w_scales[o];
            if (bias) y += bias[o];
            out[s * n + o] = y;
        }
    }
}

// normalize_strict_index_value (KC:20058-20090).
inline int64_t strict_index(double v, int64_t dim_size) {
    if (!std::isfinite(v)) return -1;
    if (std::fabs(v - std::trunc(v)) > std::numeric_limits<double>::epsilon()) return -1;
    if (v < 0.0 || v >= 9.2233720368547758e18) return -1;
    int64_t i = (int64_t)v;
    if (i < 0 || i >= dim_size) return -1;
    return i;
}

// index_select_tensor_contiguous_f32 (KC:40216-40253). Returns the position of the first
// invalid index (the reference returns Err there), or -1.
template <typename T>
int64_t index_select_impl(const T *input, int64_t outer, int64_t dim_size, int64_t inner, const double *indices,
                          int64_t n_idx, T *out) {
    for (int64_t i = 0; i < n_idx; ++i)
        if (strict_index(indices[i], dim_size) < 0) return i;
    for (int64_t o = 0; o < outer; ++o)
        for (int64_t i = 0; i < n_idx; ++i) {
            const int64_t idx = strict_index(indices[i], dim_size);
            const T *src = input + (o * dim_size + idx) * inner;
            T *dst = out + (o * n_idx + i) * inner;
            for (int64_t c = 0; c < inner; ++c) dst[c] = src[c];
        }
    return -1;
}

// argmax_dim_tensor_contiguous_f32 (KC:39443-39550), the serial lane loop KC:39518-39535:
// first strict maximum wins; the first NaN wins and ends the scan.
template <typename T> void argmax_impl(const T *x, int64_t outer, int64_t reduce, int64_t inner, T *out) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < outer * inner; ++i) {
        const int64_t o = i / inner, c = i % inner;
        const T *base = x + o * reduce * inner + c;
        int64_t best = 0;
        T best_val = -std::numeric_limits<T>::infinity();
        for (int64_t r = 0; r < reduce; ++r) {
            T val = base[r * inner];
            if (val != val) {
                best = r;
                break;
            } else if (val > best_val) {
                best_val = val;
                best = r;
            }
        }
        out[i] = (T)best;
    }
}

// permute [d0,d1,d2,d3] -> [d0,d2,d1,d3] (crates/ft-autograd/src/lib.rs:10733-10882).
template <typename T> void permute_0213_impl(const T *src, T *dst, int64_t d0, int64_t d1, int64_t d2, int64_t d3) {
#pragma omp parallel for schedule(static) collapse(2)
    for (int64_t i0 = 0; i0 < d0; ++i0)
        for (int64_t i2 = 0; i2 < d2; ++i2)
            for (int64_t i1 = 0; i1 < d1; ++i1)
                std::memcpy(dst + (((i0 * d2 + i2) * d1 + i1) * d3), src + (((i0 * d1 + i1) * d2 + i2) * d3),
                            sizeof(T) * (size_t)d3);
}

struct LayerW {
    const float *ln1_w, *ln1_b, *wq, *bq, *wk, *bk, *wv, *bv, *wo, *bo, *ln2_w, *ln2_b, *w1, *b1, *w2, *b2;
};

// TransformerEncoderLayer::forward_layer_masked with norm_first (crates/ft-nn/src/lib.rs:
// 14709-14744): x = x + MHA(LN1(x)); x = x + W2.gelu(W1.LN2(x)); MHA as
// MultiheadAttention::forward_qkv_masked (crates/ft-nn/src/lib.rs:5088-5198), scale 1/sqrt(hd).
void encoder_layer_impl(const LayerW &w, float *x, int64_t batch, int64_t seq, int64_t d_model, int64_t heads,
                        int64_t d_ff, float eps, int causal, int gelu_tanh = 0) {
    const int64_t tokens = batch * seq, hd = d_model / heads;
    std::vector<float> h((size_t)tokens * d_model), qv(h.size()), kv(h.size()), vv(h.size());
    std::vector<float> qh(h.size()), kh(h.size()), vh(h.size()), ctx(h.size()), merged(h.size()), proj(h.size());
    layer_norm_impl<float>(x, nullptr, w.ln1_w, w.ln1_b, h.data(), tokens, d_model, eps);
    linear_impl<float>(h.data(), w.wq, w.bq, tokens, d_model, d_model, qv.data());
    linear_impl<float>(h.data(), w.wk, w.bk, tokens, d_model, d_model, kv.data());
    linear_impl<float>(h.data(), w.wv, w.bv, tokens, d_model, d_model, vv.data());
    permute_0213_impl<float>(qv.data(), qh.data(), batch, seq, heads, hd);
    permute_0213_impl<float>(kv.data(), kh.data(), batch, seq, heads, hd);
    permute_0213_impl<float>(vv.data(), vh.data(), batch, seq, heads, hd);
    const float scale = (float)(1.0 / std::sqrt((double)hd));
    sdpa_impl<float>(qh.data(), kh.data(), vh.data(), batch * heads, seq, seq, hd, hd, scale, causal, ctx.data());
    permute_0213_impl<float>(ctx.data(), merged.data(), batch, heads, seq, hd);
    linear_impl<float>(merged.data(), w.wo, w.bo, tokens, d_model, d_model, proj.data());
    for (size_t i = 0; i < proj.size(); ++i) x[i] = x[i] + proj[i];
    layer_norm_impl<float>(x, nullptr, w.ln2_w, w.ln2_b, h.data(), tokens, d_model, eps);
    std::vector<float> f1((size_t)tokens * d_ff);
    linear_impl<float>(h.data(), w.w1, w.b1, tokens, d_model, d_ff, f1.data());
    for (size_t i = 0; i < f1.size(); ++i) f1[i] = gelu_tanh ? gelu_tanh_value(f1[i]) : gelu_value(f1[i]);
    linear_impl<float>(f1.data(), w.w2, w.b2, tokens, d_ff, d_model, proj.data());
    for (size_t i = 0; i < proj.size(); ++i) x[i] = x[i] + proj[i];
}

#if defined(__x86_64__)
// Blocked f32 GEMM with an AVX2/FMA 6x16 register tile, standing in for matrixmultiply's packed
// micro-kernel when the CPU path is TIMED (never used as the truth). b is [k, n].
__attribute__((target("avx2,fma"))) void sgemm_blocked_avx2(int64_t m, int64_t n, int64_t k, const float *a,
                                                            int64_t lda, const float *b, int64_t ldb, float *c,
                                                            int64_t ldc) {
    constexpr int64_t MR = 6, NR = 16, KC = 256, NC = 1024;
#pragma omp parallel
    {
        std::vector<float> bp((size_t)KC * NC);
        for (int64_t jc = 0; jc < n; jc += NC) {
            const int64_t nc = std::min(NC, n - jc);
            for (int64_t pc = 0; pc < k; pc += KC) {
                const int64_t kc = std::min(KC, k - pc);
                // every thread packs its own copy of the B panel, NR-wide column strips
                for (int64_t j0 = 0; j0 < nc; j0 += NR)
                    for (int64_t p = 0; p < kc; ++p)
                        for (int64_t j = 0; j < NR; ++j)
                            bp[(size_t)(j0 * kc + p * NR + j)] =
                                (j0 + j < nc) ? b[(pc + p) * ldb + jc + j0 + j] : 0.0f;
#pragma omp for schedule(static)
                for (int64_t i0 = 0; i0 < m; i0 += MR) {
                    const int64_t mr = std::min(MR, m - i0);
                    for (int64_t j0 = 0; j0 < nc; j0 += NR) {
                        __m256 acc[MR][2];
                        for (int r = 0; r < MR; ++r) acc[r][0] = acc[r][1] = _mm256_setzero_ps();
                        const float *bs = bp.data() + j0 * kc;
                        for (int64_t p = 0; p < kc; ++p) {
                            const __m256 b0 = _mm256_loadu_ps(bs + p * NR), b1 = _mm256_loadu_ps(bs + p * NR + 8);
                            for (int r = 0; r < MR; ++r) {
                                const float av = (r < mr) ? a[(i0 + r) * lda + pc + p] : 0.0f;
                                const __m256 ab = _mm256_set1_ps(av);
                                acc[r][0] = _mm256_fmadd_ps(ab, b0, acc[r][0]);
                                acc[r][1] = _mm256_fmadd_ps(ab, b1, acc[r][1]);
                            }
                        }
                        float tmp[NR];
                        for (int r = 0; r < mr; ++r) {
                            _mm256_storeu_ps(tmp, acc[r][0]);
                            _mm256_storeu_ps(tmp + 8, acc[r][1]);
                            float *cr = c + (i0 + r) * ldc + jc + j0;
                            const int64_t w = std::min<int64_t>(NR, nc - j0);
                            if (pc == 0) for (int64_t j = 0; j < w; ++j) cr[j] = tmp[j];
                            else for (int64_t j = 0; j < w; ++j) cr[j] += tmp[j];
                        }
                    }
                }
            }
        }
    }
}
#endif

}  // namespace

// log_softmax_dim_tensor_contiguous_f32 (KC:39298-39375), _f64 (KC:18504-18590): per lane,
// max = fold(-inf, max); sum_exp = pairwise_sum(exp(x - max)); out = (x - max) - ln(sum_exp).
inline float t_log(float x) { return logf(x); }
inline double t_log(double x) { return log(x); }
template <typename T> void log_softmax_impl(const T *x, T *y, int64_t outer, int64_t reduce, int64_t inner) {
    if (outer <= 0 || reduce <= 0 || inner <= 0) return;
#pragma omp parallel
    {
        std::vector<T> scratch((size_t)reduce), ex((size_t)reduce);
#pragma omp for schedule(static) collapse(2)
        for (int64_t o = 0; o < outer; ++o) {
            for (int64_t c = 0; c < inner; ++c) {
                const T *in = x + o * reduce * inner + c;
                T *out = y + o * reduce * inner + c;
                for (int64_t r = 0; r < reduce; ++r) scratch[r] = in[r * inner];
                T m = -std::numeric_limits<T>::infinity();
                for (int64_t r = 0; r < reduce; ++r) m = max_num(m, scratch[r]);
                for (int64_t r = 0; r < reduce; ++r) ex[r] = t_exp(scratch[r] - m);
                const T lse = t_log(pairwise_sum(ex.data(), (size_t)reduce));
                for (int64_t r = 0; r < reduce; ++r) out[r * inner] = (scratch[r] - m) - lse;
            }
        }
    }
}

// cross_entropy_forward_f32 / _f64 (KC:6717-6738, 6649-6671): strict `>` max scan, sequential sum of
// exp(v - m), lse = m + ln(s), loss = lse - row[target]. Returns the first row with an invalid target, or -1.
template <typename T> int64_t cross_entropy_forward_impl(const T *logits, const int64_t *target, int64_t batch, int64_t classes, T *loss) {
    int64_t bad = -1;
    for (int64_t i = 0; i < batch; ++i)
        if (target[i] < 0 || target[i] >= classes) {
            bad = i;
            break;
        }
    if (bad >= 0) return bad;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < batch; ++i) {
        const T *row = logits + i * classes;
        T m = -std::numeric_limits<T>::infinity();
        for (int64_t c = 0; c < classes; ++c)
            if (row[c] > m) m = row[c];
        T s = 0;
        for (int64_t c = 0; c < classes; ++c) s += t_exp(row[c] - m);
        loss[i] = (m + t_log(s)) - row[target[i]];
    }
    return -1;
}

// cross_entropy_backward_f32 / _f64 (KC:6745-6781, 6679-6712): dlogits[i][c] = dloss[i] * (exp(row[c] - lse) - [c == target[i]]).
template <typename T>
int64_t cross_entropy_backward_impl(const T *logits, const int64_t *target, const T *dloss, int64_t batch, int64_t classes, T *dlogits) {
    for (int64_t i = 0; i < batch; ++i)
        if (target[i] < 0 || target[i] >= classes) return i;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < batch; ++i) {
        const T *row = logits + i * classes;
        T m = -std::numeric_limits<T>::infinity();
        for (int64_t c = 0; c < classes; ++c)
            if (row[c] > m) m = row[c];
        T s = 0;
        for (int64_t c = 0; c < classes; ++c) s += t_exp(row[c] - m);
        const T lse = m + t_log(s), g = dloss[i];
        for (int64_t c = 0; c < classes; ++c) dlogits[i * classes + c] = g * (t_exp(row[c] - lse) - (c == target[i] ? T(1) : T(0)));
    }
    return -1;
}

// ------------------------------------------------------------------------------------------
// Backward kernels of the same ops (the rows the forward path widens into next).

// layer_norm_backward_f32 / _f64 (KC:6189-6322, 6052-6183): recomputes mean / rstd per row with the
// forward's sequential sums, c1 = sum_j dxhat, c2 = sum_j dxhat * xhat,
// dx = rstd * (dxhat - (c1 + xhat * c2) * inv_n); dweight / dbias are serial sums over the rows.
// (The unit-dy shortcut KC:6198-6254 computes the same values with dy = 1 and is not restated.)
template <typename T>
void layer_norm_backward_impl(const T *dy, const T *x, const T *w, int64_t batch, int64_t n, T eps, T *dx, T *dw, T *db) {
    const T inv_n = T(1) / (T)n;
    std::vector<T> means((size_t)std::max<int64_t>(batch, 1)), rstds((size_t)std::max<int64_t>(batch, 1));
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < batch; ++r) {
        const T *xr = x + r * n, *dyr = dy + r * n;
        T sum = 0;
        for (int64_t j = 0; j < n; ++j) sum += xr[j];
        const T mean = sum * inv_n;
        T vsum = 0;
        for (int64_t j = 0; j < n; ++j) {
            const T d = xr[j] - mean;
            vsum += d * d;
        }
        const T rstd = T(1) / std::sqrt(vsum * inv_n + eps);
        means[(size_t)r] = mean;
        rstds[(size_t)r] = rstd;
        T c1 = 0, c2 = 0;
        for (int64_t j = 0; j < n; ++j) {
            const T xhat = (xr[j] - mean) * rstd;
            const T dxhat = dyr[j] * w[j];
            c1 += dxhat;
            c2 += dxhat * xhat;
        }
        for (int64_t j = 0; j < n; ++j) {
            const T xhat = (xr[j] - mean) * rstd;
            const T dxhat = dyr[j] * w[j];
            dx[r * n + j] = rstd * (dxhat - (c1 + xhat * c2) * inv_n);
        }
    }
    for (int64_t j = 0; j < n; ++j) dw[j] = db[j] = 0;
    for (int64_t r = 0; r < batch; ++r) {
        const T *xr = x + r * n, *dyr = dy + r * n;
        const T mean = means[(size_t)r], rstd = rstds[(size_t)r];
        for (int64_t j = 0; j < n; ++j) {
            const T xhat = (xr[j] - mean) * rstd;
            dw[j] += dyr[j] * xhat;
            db[j] += dyr[j];
        }
    }
}

// rms_norm_backward_f32 / _f64 (KC:6574-6646, 6503-6570): g = dy * w (w optional),
// rstd = 1 / sqrt(mean(x^2) + eps), c = sum_j g * x, dx = rstd * g - (rstd^3 * c / n) * x,
// dweight[j] = sum_rows dy * x * rstd (serial over the rows), only when a weight is given.
template <typename T>
void rms_norm_backward_impl(const T *dy, const T *x, const T *w, int64_t batch, int64_t n, T eps, T *dx, T *dw) {
    const T inv_n = T(1) / (T)n;
    std::vector<T> rstds((size_t)std::max<int64_t>(batch, 1));
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < batch; ++r) {
        const T *xr = x + r * n, *dyr = dy + r * n;
        T ss = 0;
        for (int64_t j = 0; j < n; ++j) ss += xr[j] * xr[j];
        const T rstd = T(1) / std::sqrt(ss * inv_n + eps);
        rstds[(size_t)r] = rstd;
        T c = 0;
        for (int64_t j = 0; j < n; ++j) {
            const T g = dyr[j] * (w ? w[j] : T(1));
            c += g * xr[j];
        }
        const T coef = rstd * rstd * rstd * c * inv_n;
        for (int64_t j = 0; j < n; ++j) {
            const T g = dyr[j] * (w ? w[j] : T(1));
            dx[r * n + j] = rstd * g - coef * xr[j];
        }
    }
    if (w && dw) {
        for (int64_t j = 0; j < n; ++j) dw[j] = 0;
        for (int64_t r = 0; r < batch; ++r) {
            const T *xr = x + r * n, *dyr = dy + r * n;
            const T rstd = rstds[(size_t)r];
            for (int64_t j = 0; j < n; ++j) dw[j] += dyr[j] * xr[j] * rstd;
        }
    }
}

// Wide-accumulation product with A stored [k, m] (gemm::sgemm_tb / dgemm_tb, KC:1484-1524, 262-345).
template <typename T> void gemm_tb_any(int64_t m, int64_t n, int64_t k, T alpha, const T *a_km, const T *b_kn, T *c) {
    if (m <= 0 || n <= 0) return;
    std::vector<T> at((size_t)m * (size_t)std::max<int64_t>(k, 1));
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; ++i)
        for (int64_t p = 0; p < k; ++p) at[(size_t)i * k + p] = a_km[p * m + i];
    gemm_any(0, m, n, k, at.data(), k, b_kn, n, c, n);
    if (alpha != T(1))
        for (int64_t i = 0; i < m * n; ++i) c[i] = alpha * c[i];
}

// linear_backward_f64 (KC:17226-17302) and its f32 twin by the same formulas:
// dx = dy . W ([batch,out] . [out,in]), dweight = dy^T . x, dbias = serial sum of dy over the rows.
template <typename T>
void linear_backward_impl(const T *dy, const T *x, const T *w, int64_t batch, int64_t in_f, int64_t out_f, T *dx, T *dw, T *db) {
    if (batch > 0 && in_f > 0) gemm_any(0, batch, in_f, out_f, dy, out_f, w, in_f, dx, in_f);
    if (out_f > 0 && in_f > 0) gemm_tb_any<T>(out_f, in_f, batch, T(1), dy, x, dw);
    if (db) {
        for (int64_t o = 0; o < out_f; ++o) db[o] = 0;
        for (int64_t b = 0; b < batch; ++b)
            for (int64_t o = 0; o < out_f; ++o) db[o] += dy[b * out_f + o];
    }
}

// sdpa_backward_f32 / _f64 (KC:5539-5650, 5300-5414): per (batch*head) P = softmax(scale * Q.K^T)
// with the forward's row loop (strict max scan over the first `limit` entries, exp, sequential
// sum, divide, zero tail), dU = dOut.V^T, dot_i = sum_j P_ij dU_ij, dU_ij = P_ij (dU_ij - dot_i),
// dV = P^T.dOut, dQ = scale * dU.K, dK = scale * dU^T.Q. The products are the wide-accumulation
// truth; the alpha of the scaled products is applied to the rounded product.
// sdpa_backward_masked_f64 (KC:5423-5530) is the same with the score s * scale + mask[bh * mask_bh_stride + i * seq_k + j]
// (KC:5466-5475) and no causal limit; `mask` non-NULL selects it.
template <typename T>
void sdpa_backward_impl(const T *q, const T *k, const T *v, const T *dout, int64_t num_bh, int64_t seq_q, int64_t seq_k,
                        int64_t d_k, int64_t d_v, T scale, int causal, T *dq, T *dk, T *dv, const T *mask = nullptr,
                        int64_t mask_bh_stride = 0) {
    std::vector<T> p((size_t)std::max<int64_t>(seq_q * seq_k, 1)), du((size_t)std::max<int64_t>(seq_q * seq_k, 1));
    for (int64_t bh = 0; bh < num_bh; ++bh) {
        const T *qh = q + bh * seq_q * d_k, *kh = k + bh * seq_k * d_k, *vh = v + bh * seq_k * d_v;
        const T *doh = dout + bh * seq_q * d_v;
        T *dqh = dq + bh * seq_q * d_k, *dkh = dk + bh * seq_k * d_k, *dvh = dv + bh * seq_k * d_v;
        if (seq_q > 0 && seq_k > 0) gemm_any(1, seq_q, seq_k, d_k, qh, d_k, kh, d_k, p.data(), seq_k);
        for (int64_t i = 0; i < seq_q; ++i) {
            const int64_t limit = causal ? std::min<int64_t>(i + 1, seq_k) : seq_k;
            T *row = p.data() + i * seq_k;
            T m = -std::numeric_limits<T>::infinity();
            const T *mrow = mask ? mask + bh * mask_bh_stride + i * seq_k : nullptr;
            for (int64_t j = 0; j < limit; ++j) {
                row[j] = mrow ? row[j] * scale + mrow[j] : row[j] * scale;
                if (row[j] > m) m = row[j];
            }
            T sum = 0;
            for (int64_t j = 0; j < limit; ++j) {
                const T e = std::exp(row[j] - m);
                row[j] = e;
                sum += e;
            }
            for (int64_t j = 0; j < limit; ++j) row[j] /= sum;
            for (int64_t j = limit; j < seq_k; ++j) row[j] = 0;
        }
        if (seq_q > 0 && seq_k > 0) gemm_any(1, seq_q, seq_k, d_v, doh, d_v, vh, d_v, du.data(), seq_k);
        for (int64_t i = 0; i < seq_q; ++i) {
            const T *pr = p.data() + i * seq_k;
            T *dr = du.data() + i * seq_k;
            T dot = 0;
            for (int64_t j = 0; j < seq_k; ++j) dot += pr[j] * dr[j];
            for (int64_t j = 0; j < seq_k; ++j) dr[j] = pr[j] * (dr[j] - dot);
        }
        gemm_tb_any<T>(seq_k, d_v, seq_q, T(1), p.data(), doh, dvh);
        if (seq_q > 0 && d_k > 0) {
            gemm_any(0, seq_q, d_k, seq_k, du.data(), seq_k, kh, d_k, dqh, d_k);
            for (int64_t i = 0; i < seq_q * d_k; ++i) dqh[i] = scale * dqh[i];
        }
        gemm_tb_any<T>(seq_k, d_k, seq_q, scale, du.data(), qh, dkh);
    }
}

// sdpa_backward_f32_unit_dout (KC:5662-5770): dOut = ones without materialising it. dP_ij = sum_l V_jl (sequential), the
// dot and dU rows from it, dV_jl = sum_i P_ij for every l (accumulated row by row), dQ / dK as in the general form.
template <typename T>
void sdpa_backward_unit_dout_impl(const T *q, const T *k, const T *v, int64_t num_bh, int64_t seq_q, int64_t seq_k, int64_t d_k, int64_t d_v,
                                  T scale, int causal, T *dq, T *dk, T *dv) {
    std::vector<T> p((size_t)std::max<int64_t>(seq_q * seq_k, 1)), du((size_t)std::max<int64_t>(seq_q * seq_k, 1));
    std::vector<T> vrs((size_t)std::max<int64_t>(seq_k, 1)), pcs((size_t)std::max<int64_t>(seq_k, 1));
    for (int64_t bh = 0; bh < num_bh; ++bh) {
        const T *qh = q + bh * seq_q * d_k, *kh = k + bh * seq_k * d_k, *vh = v + bh * seq_k * d_v;
        T *dqh = dq + bh * seq_q * d_k, *dkh = dk + bh * seq_k * d_k, *dvh = dv + bh * seq_k * d_v;
        if (seq_q > 0 && seq_k > 0) gemm_any(1, seq_q, seq_k, d_k, qh, d_k, kh, d_k, p.data(), seq_k);
        for (int64_t i = 0; i < seq_q; ++i) {
            const int64_t limit = causal ? std::min<int64_t>(i + 1, seq_k) : seq_k;
            T *row = p.data() + i * seq_k;
            T m = -std::numeric_limits<T>::infinity();
            for (int64_t j = 0; j < limit; ++j) {
                row[j] *= scale;
                if (row[j] > m) m = row[j];
            }
            T sum = 0;
            for (int64_t j = 0; j < limit; ++j) {
                const T e = std::exp(row[j] - m);
                row[j] = e;
                sum += e;
            }
            for (int64_t j = 0; j < limit; ++j) row[j] /= sum;
            for (int64_t j = limit; j < seq_k; ++j) row[j] = 0;
        }
        for (int64_t j = 0; j < seq_k; ++j) {
            T sum = 0;
            for (int64_t l = 0; l < d_v; ++l) sum += vh[j * d_v + l];
            vrs[j] = sum;
            pcs[j] = 0;
        }
        for (int64_t i = 0; i < seq_q; ++i) {
            const T *pr = p.data() + i * seq_k;
            T *dr = du.data() + i * seq_k;
            T dot = 0;
            for (int64_t j = 0; j < seq_k; ++j) dot += pr[j] * vrs[j];
            for (int64_t j = 0; j < seq_k; ++j) {
                dr[j] = pr[j] * (vrs[j] - dot);
                pcs[j] += pr[j];
            }
        }
        for (int64_t j = 0; j < seq_k; ++j)
            for (int64_t l = 0; l < d_v; ++l) dvh[j * d_v + l] = pcs[j];
        if (seq_q > 0 && d_k > 0) {
            gemm_any(0, seq_q, d_k, seq_k, du.data(), seq_k, kh, d_k, dqh, d_k);
            for (int64_t i = 0; i < seq_q * d_k; ++i) dqh[i] = scale * dqh[i];
        }
        gemm_tb_any<T>(seq_k, d_k, seq_q, scale, du.data(), qh, dkh);
    }
}

extern "C" {

void fto_log_softmax_f32(const float *x, float *y, int64_t outer, int64_t reduce, int64_t inner) {
    log_softmax_impl<float>(x, y, outer, reduce, inner);
}
void fto_log_softmax_f64(const double *x, double *y, int64_t outer, int64_t reduce, int64_t inner) {
    log_softmax_impl<double>(x, y, outer, reduce, inner);
}
int64_t fto_cross_entropy_forward_f32(const float *logits, const int64_t *target, int64_t batch, int64_t classes, float *loss) {
    return cross_entropy_forward_impl<float>(logits, target, batch, classes, loss);
}
int64_t fto_cross_entropy_forward_f64(const double *logits, const int64_t *target, int64_t batch, int64_t classes, double *loss) {
    return cross_entropy_forward_impl<double>(logits, target, batch, classes, loss);
}
int64_t fto_cross_entropy_backward_f32(const float *logits, const int64_t *target, const float *dloss, int64_t batch, int64_t classes,
                                       float *dlogits) {
    return cross_entropy_backward_impl<float>(logits, target, dloss, batch, classes, dlogits);
}
int64_t fto_cross_entropy_backward_f64(const double *logits, const int64_t *target, const double *dloss, int64_t batch, int64_t classes,
                                       double *dlogits) {
    return cross_entropy_backward_impl<double>(logits, target, dloss, batch, classes, dlogits);
}

void fto_layer_norm_backward_f32(const float *dy, const float *x, const float *w, int64_t batch, int64_t n, float eps,
                                 float *dx, float *dw, float *db) {
    layer_norm_backward_impl<float>(dy, x, w, batch, n, eps, dx, dw, db);
}
void fto_layer_norm_backward_f64(const double *dy, const double *x, const double *w, int64_t batch, int64_t n, double eps,
                                 double *dx, double *dw, double *db) {
    layer_norm_backward_impl<double>(dy, x, w, batch, n, eps, dx, dw, db);
}
void fto_rms_norm_backward_f32(const float *dy, const float *x, const float *w, int64_t batch, int64_t n, float eps,
                               float *dx, float *dw) {
    rms_norm_backward_impl<float>(dy, x, w, batch, n, eps, dx, dw);
}
void fto_rms_norm_backward_f64(const double *dy, const double *x, const double *w, int64_t batch, int64_t n, double eps,
                               double *dx, double *dw) {
    rms_norm_backward_impl<double>(dy, x, w, batch, n, eps, dx, dw);
}
void fto_linear_backward_f32(const float *dy, const float *x, const float *w, int64_t batch, int64_t in_f, int64_t out_f,
                             float *dx, float *dw, float *db) {
    linear_backward_impl<float>(dy, x, w, batch, in_f, out_f, dx, dw, db);
}
void fto_linear_backward_f64(const double *dy, const double *x, const double *w, int64_t batch, int64_t in_f, int64_t out_f,
                             double *dx, double *dw, double *db) {
    linear_backward_impl<double>(dy, x, w, batch, in_f, out_f, dx, dw, db);
}
void fto_sdpa_backward_f32(const float *q, const float *k, const float *v, const float *dout, int64_t num_bh, int64_t seq_q,
                           int64_t seq_k, int64_t d_k, int64_t d_v, float scale, int causal, float *dq, float *dk, float *dv) {
    sdpa_backward_impl<float>(q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, causal, dq, dk, dv);
}
void fto_sdpa_backward_unit_dout_f32(const float *q, const float *k, const float *v, int64_t num_bh, int64_t seq_q, int64_t seq_k, int64_t d_k,
                                     int64_t d_v, float scale, int causal, float *dq, float *dk, float *dv) {
    sdpa_backward_unit_dout_impl<float>(q, k, v, num_bh, seq_q, seq_k, d_k, d_v, scale, causal, dq, dk, dv);
}
void fto_sdpa_backward_unit_dout_f64(const double *q, const double *k, const double *v, int64_t num_bh, int64_t seq_q, int64_t seq_k, int64_t d_k,
                                     int64_t d_v, double scale, int causal, double *dq, double *dk, double *dv) {
    sdpa_backward_unit_dout_impl<double>(q, k, v, num_bh, seq_q, seq_k, d_k, d_v, scale, causal, dq, dk, dv);
}
void fto_sdpa_backward_masked_f32(const float *q, const float *k, const float *v, const float *dout, int64_t num_bh, int64_t seq_q,
                                  int64_t seq_k, int64_t d_k, int64_t d_v, float scale, const float *mask, int64_t mask_bh_stride, float *dq,
                                  float *dk, float *dv) {
    sdpa_backward_impl<float>(q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, 0, dq, dk, dv, mask, mask_bh_stride);
}
void fto_sdpa_backward_masked_f64(const double *q, const double *k, const double *v, const double *dout, int64_t num_bh, int64_t seq_q,
                                  int64_t seq_k, int64_t d_k, int64_t d_v, double scale, const double *mask, int64_t mask_bh_stride,
                                  double *dq, double *dk, double *dv) {
    sdpa_backward_impl<double>(q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, 0, dq, dk, dv, mask, mask_bh_stride);
}
void fto_sdpa_backward_f64(const double *q, const double *k, const double *v, const double *dout, int64_t num_bh,
                           int64_t seq_q, int64_t seq_k, int64_t d_k, int64_t d_v, double scale, int causal, double *dq,
                           double *dk, double *dv) {
    sdpa_backward_impl<double>(q, k, v, dout, num_bh, seq_q, seq_k, d_k, d_v, scale, causal, dq, dk, dv);
}

void fto_softmax_f32(const float *x, float *y, int64_t outer, int64_t reduce, int64_t inner) {
    softmax_impl<float>(x, y, outer, reduce, inner);
}
void fto_softmax_f64(const double *x, double *y, int64_t outer, int64_t reduce, int64_t inner) {
    softmax_impl<double>(x, y, outer, reduce, inner);
}
void fto_layer_norm_f32(const float *x, const float *w, const float *b, float *y, int64_t batch, int64_t n, float eps) {
    layer_norm_impl<float>(x, nullptr, w, b, y, batch, n, eps);
}
void fto_layer_norm_f64(const double *x, const double *w, const double *b, double *y, int64_t batch, int64_t n,
                        double eps) {
    layer_norm_impl<double>(x, nullptr, w, b, y, batch, n, eps);
}
void fto_add_layer_norm_f32(const float *a, const float *b2, const float *w, const float *b, float *y, int64_t batch,
                            int64_t n, float eps) {
    layer_norm_impl<float>(a, b2, w, b, y, batch, n, eps);
}
void fto_rms_norm_f32(const float *x, const float *w, float *y, int64_t batch, int64_t n, float eps) {
    rms_norm_impl<float>(x, w, y, batch, n, eps);
}
void fto_rms_norm_f64(const double *x, const double *w, double *y, int64_t batch, int64_t n, double eps) {
    rms_norm_impl<double>(x, w, y, batch, n, eps);
}
// gelu_tensor_contiguous_f32 (KC:37123-37127)
void fto_gelu_f32(const float *x, float *y, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) y[i] = gelu_value(x[i]);
}
void fto_gelu_tanh_f32(const float *x, float *y, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) y[i] = gelu_tanh_value(x[i]);
}
void fto_gelu_tanh_f64(const double *x, double *y, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) y[i] = gelu_tanh_value(x[i]);
}
void fto_gelu_f64(const double *x, double *y, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) y[i] = gelu_value(x[i]);
}
// add_tensor_contiguous_f32 (KC:36870-36877)
void fto_add_f32(const float *a, const float *b, float *y, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) y[i] = a[i] + b[i];
}
void fto_add_f64(const double *a, const double *b, double *y, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) y[i] = a[i] + b[i];
}
// bias pass of linear_tensor_f32 (KC:17336-17351), optionally followed by the residual add
void fto_bias_add_f32(const float *x, const float *bias, const float *residual, float *y, int64_t rows, int64_t cols) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t j = 0; j < cols; ++j) {
            float v = x[r * cols + j] + bias[j];
            if (residual) v = v + residual[r * cols + j];
            y[r * cols + j] = v;
        }
}
void fto_bias_add_f64(const double *x, const double *bias, const double *residual, double *y, int64_t rows,
                      int64_t cols) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t j = 0; j < cols; ++j) {
            double v = x[r * cols + j] + bias[j];
            if (residual) v = v + residual[r * cols + j];
            y[r * cols + j] = v;
        }
}

// gemm::sgemm / sgemm_bt (KC:1310-1338, 1430-1481) and dgemm / dgemm_bt (KC:107-138, 201-255)
void fto_gemm_f32(int trans_b, int64_t m, int64_t n, int64_t k, const float *a, int64_t lda, const float *b,
                  int64_t ldb, float *c, int64_t ldc) {
    gemm_any(trans_b, m, n, k, a, lda, b, ldb, c, ldc);
}
void fto_gemm_f64(int trans_b, int64_t m, int64_t n, int64_t k, const double *a, int64_t lda, const double *b,
                  int64_t ldb, double *c, int64_t ldc) {
    gemm_any(trans_b, m, n, k, a, lda, b, ldb, c, ldc);
}
// Timed stand-in for matrixmultiply (not a truth): returns 0 when AVX2/FMA is unavailable.
int fto_sgemm_blocked(int64_t m, int64_t n, int64_t k, const float *a, int64_t lda, const float *b, int64_t ldb,
                      float *c, int64_t ldc) {
#if defined(__x86_64__)
    if (__builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma")) {
        sgemm_blocked_avx2(m, n, k, a, lda, b, ldb, c, ldc);
        return 1;
    }
#endif
    return 0;
}
// bmm_tensor_contiguous_f32 (KC:38496-38606): per-batch sgemm
void fto_bmm_f32(int64_t batch, int64_t m, int64_t n, int64_t k, const float *a, const float *b, float *c) {
    for (int64_t i = 0; i < batch; ++i) gemm_any(0, m, n, k, a + i * m * k, k, b + i * k * n, n, c + i * m * n, n);
}
void fto_bmm_f64(int64_t batch, int64_t m, int64_t n, int64_t k, const double *a, const double *b, double *c) {
    for (int64_t i = 0; i < batch; ++i) gemm_any(0, m, n, k, a + i * m * k, k, b + i * k * n, n, c + i * m * n, n);
}
// addmm_tensor_contiguous_f32 (KC:41562-41648): beta * input_at(i) + alpha * g, input [n] or [m,n]
void fto_addmm_f32(const float *input, int input_is_1d, const float *mat1, const float *mat2, int64_t m, int64_t n,
                   int64_t k, float beta, float alpha, float *out) {
    uint32_t abits;
    std::memcpy(&abits, &alpha, 4);
    if (abits == 0) {
        for (int64_t i = 0; i < m * n; ++i) out[i] = beta * (input_is_1d ? input[i % n] : input[i]);
        return;
    }
    std::vector<float> g((size_t)(m * n));
    gemm_any(0, m, n, k, mat1, k, mat2, n, g.data(), n);
    for (int64_t i = 0; i < m * n; ++i) out[i] = beta * (input_is_1d ? input[i % n] : input[i]) + alpha * g[i];
}
void fto_addmm_f64(const double *input, int input_is_1d, const double *mat1, const double *mat2, int64_t m,
                   int64_t n, int64_t k, double beta, double alpha, double *out) {
    uint64_t abits;
    std::memcpy(&abits, &alpha, 8);
    if (abits == 0) {
        for (int64_t i = 0; i < m * n; ++i) out[i] = beta * (input_is_1d ? input[i % n] : input[i]);
        return;
    }
    std::vector<double> g((size_t)(m * n));
    gemm_any(0, m, n, k, mat1, k, mat2, n, g.data(), n);
    for (int64_t i = 0; i < m * n; ++i) out[i] = beta * (input_is_1d ? input[i % n] : input[i]) + alpha * g[i];
}
void fto_linear_f32(const float *x, const float *w, const float *bias, int64_t batch, int64_t in_f, int64_t out_f,
                    float *y) {
    linear_impl<float>(x, w, bias, batch, in_f, out_f, y);
}
void fto_linear_f64(const double *x, const double *w, const double *bias, int64_t batch, int64_t in_f, int64_t out_f,
                    double *y) {
    linear_impl<double>(x, w, bias, batch, in_f, out_f, y);
}
void fto_sdpa_forward_f32(const float *q, const float *k, const float *v, int64_t num_bh, int64_t seq_q,
                          int64_t seq_k, int64_t d_k, int64_t d_v, float scale, int causal, float *out) {
    sdpa_impl<float>(q, k, v, num_bh, seq_q, seq_k, d_k, d_v, scale, causal, out);
}
void fto_quantize_rows_i8(const float *x, int64_t rows, int64_t cols, int8_t *q, float *scales) { quantize_rows_i8_impl(x, rows, cols, q, scales); }
void fto_linear_int8_dynamic_f32(const float *x, int64_t m, int64_t k, const int8_t *w_i8, const float *w_scales, int64_t n, const float *bias,
                                 float *out) {
    linear_int8_dynamic_impl(x, m, k, w_i8, w_scales, n, bias, out);
}
void fto_sdpa_forward_masked_gqa_f32(const float *q, const float *k, const float *v, int64_t batch, int64_t h_q, int64_t h_kv,
                                     int64_t seq_q, int64_t seq_k, int64_t d_k, int64_t d_v, float scale, const float *mask,
                                     int64_t mask_bh_stride, float *out) {
    sdpa_masked_gqa_impl<float>(q, k, v, batch, h_q, h_kv, seq_q, seq_k, d_k, d_v, scale, mask, mask_bh_stride, out);
}
void fto_sdpa_forward_masked_gqa_f64(const double *q, const double *k, const double *v, int64_t batch, int64_t h_q, int64_t h_kv,
                                     int64_t seq_q, int64_t seq_k, int64_t d_k, int64_t d_v, double scale, const double *mask,
                                     int64_t mask_bh_stride, double *out) {
    sdpa_masked_gqa_impl<double>(q, k, v, batch, h_q, h_kv, seq_q, seq_k, d_k, d_v, scale, mask, mask_bh_stride, out);
}
void fto_sdpa_forward_f64(const double *q, const double *k, const double *v, int64_t num_bh, int64_t seq_q,
                          int64_t seq_k, int64_t d_k, int64_t d_v, double scale, int causal, double *out) {
    sdpa_impl<double>(q, k, v, num_bh, seq_q, seq_k, d_k, d_v, scale, causal, out);
}
int64_t fto_index_select_f32(const float *input, int64_t outer, int64_t dim_size, int64_t inner,
                             const double *indices, int64_t n_idx, float *out) {
    return index_select_impl<float>(input, outer, dim_size, inner, indices, n_idx, out);
}
int64_t fto_index_select_f64(const double *input, int64_t outer, int64_t dim_size, int64_t inner,
                             const double *indices, int64_t n_idx, double *out) {
    return index_select_impl<double>(input, outer, dim_size, inner, indices, n_idx, out);
}
void fto_argmax_f32(const float *x, int64_t outer, int64_t reduce, int64_t inner, float *out) {
    argmax_impl<float>(x, outer, reduce, inner, out);
}
void fto_argmax_f64(const double *x, int64_t outer, int64_t reduce, int64_t inner, double *out) {
    argmax_impl<double>(x, outer, reduce, inner, out);
}
void fto_permute_0213_f32(const float *src, float *dst, int64_t d0, int64_t d1, int64_t d2, int64_t d3) {
    permute_0213_impl<float>(src, dst, d0, d1, d2, d3);
}
void fto_permute_0213_f64(const double *src, double *dst, int64_t d0, int64_t d1, int64_t d2, int64_t d3) {
    permute_0213_impl<double>(src, dst, d0, d1, d2, d3);
}

// One pre-LN block, in place on x [batch*seq, d_model]. `w` is 16 pointers in the order of LayerW.
void fto_encoder_layer_f32(const float *const *w, float *x, int64_t batch, int64_t seq, int64_t d_model,
                           int64_t heads, int64_t d_ff, float eps, int causal) {
    LayerW lw = {w[0], w[1], w[2], w[3], w[4], w[5], w[6], w[7], w[8], w[9], w[10], w[11], w[12], w[13], w[14], w[15]};
    encoder_layer_impl(lw, x, batch, seq, d_model, heads, d_ff, eps, causal);
}
// The same block with the tanh-form GELU (what the Metal encoder computes, fused.rs:301-313).
void fto_encoder_layer_gelu_tanh_f32(const float *const *w, float *x, int64_t batch, int64_t seq, int64_t d_model,
                                     int64_t heads, int64_t d_ff, float eps, int causal) {
    LayerW lw = {w[0], w[1], w[2], w[3], w[4], w[5], w[6], w[7], w[8], w[9], w[10], w[11], w[12], w[13], w[14], w[15]};
    encoder_layer_impl(lw, x, batch, seq, d_model, heads, d_ff, eps, causal, 1);
}

// GPT-2-shaped forward: x = wte[ids] + wpe[pos] (Embedding::forward, crates/ft-nn/src/lib.rs:
// 3080-3135, twice, then add); n_layers pre-LN causal blocks; final LayerNorm; logits = x . wte^T
// (tied head); argmax over the vocabulary. `layers` is n_layers * 16 pointers. `hidden`
// (tokens * d_model), `logits` (tokens * vocab) and `argmax` (tokens) may each be NULL.
// Returns the position of the first invalid token id, or -1.
int64_t fto_gpt2_forward_f32(int64_t vocab, int64_t max_pos, int64_t d_model, int64_t heads, int64_t d_ff, float eps,
                             const float *wte, const float *wpe, const float *const *layers, int64_t n_layers,
                             const float *lnf_w, const float *lnf_b, const double *ids, int64_t batch, int64_t seq,
                             float *hidden, float *logits, float *argmax) {
    const int64_t tokens = batch * seq;
    if (seq > max_pos) return 0;
    std::vector<float> x((size_t)tokens * d_model), tok((size_t)tokens * d_model), pos((size_t)tokens * d_model);
    int64_t bad = index_select_impl<float>(wte, 1, vocab, d_model, ids, tokens, tok.data());
    if (bad >= 0) return bad;
    std::vector<double> pidx((size_t)tokens);
    for (int64_t t = 0; t < tokens; ++t) pidx[t] = (double)(t % seq);
    index_select_impl<float>(wpe, 1, max_pos, d_model, pidx.data(), tokens, pos.data());
    for (size_t i = 0; i < x.size(); ++i) x[i] = tok[i] + pos[i];
    for (int64_t l = 0; l < n_layers; ++l) {
        const float *const *w = layers + l * 16;
        LayerW lw = {w[0], w[1], w[2], w[3], w[4], w[5], w[6], w[7], w[8], w[9], w[10], w[11], w[12], w[13], w[14], w[15]};
        encoder_layer_impl(lw, x.data(), batch, seq, d_model, heads, d_ff, eps, 1);
    }
    std::vector<float> hf(x.size());
    layer_norm_impl<float>(x.data(), nullptr, lnf_w, lnf_b, hf.data(), tokens, d_model, eps);
    if (hidden) std::memcpy(hidden, hf.data(), hf.size() * sizeof(float));
    if (logits || argmax) {
        std::vector<float> own;
        float *lg = logits;
        if (!lg) {
            own.resize((size_t)tokens * vocab);
            lg = own.data();
        }
        linear_impl<float>(hf.data(), wte, nullptr, tokens, d_model, vocab, lg);
        if (argmax) argmax_impl<float>(lg, tokens, vocab, 1, argmax);
    }
    return -1;
}

}  // extern "C"
