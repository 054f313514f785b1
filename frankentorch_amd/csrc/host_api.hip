// Tier A of the C ABI: host slices in, caller-provided host buffer out -- the call shape of the
// `ft_kernel_cpu::*` free functions that ft-dispatch routes to (crates/ft-dispatch/src/lib.rs:
// 14-250). Every function validates exactly as its reference counterpart does (same checks, same
// order, same error variant and payload), then uploads, launches the device-pointer kernels on
// the library stream, downloads and synchronises. There is no CPU computation here.

#include <cmath>
#include <limits>
#include <type_traits>

#include "common.hpp"
#include "pool.hpp"
#include "staging.hpp"

namespace {

using fth::set_error;

// ---- TensorMeta semantics (crates/ft-core/src/lib.rs:340-348, 575-607) ------------------------
bool meta_ok(const fth_meta *m) { return m && m->ndim >= 0 && m->ndim <= FTH_MAX_DIMS; }

// saturated_numel: product of the shape, saturating (the cached `numel` field).
uint64_t meta_numel(const fth_meta *m) {
    uint64_t n = 1;
    for (int i = 0; i < m->ndim; ++i) {
        if (__builtin_mul_overflow(n, m->shape[i], &n)) return std::numeric_limits<uint64_t>::max();
    }
    return n;
}

// TensorMeta::is_contiguous: size-1 dims are contiguous whatever their stride.
bool meta_contiguous(const fth_meta *m) {
    uint64_t expected = 1;
    for (int i = m->ndim - 1; i >= 0; --i) {
        if (m->shape[i] == 1) continue;
        if (m->strides[i] != expected) return false;
        if (__builtin_mul_overflow(expected, m->shape[i], &expected)) return false;
    }
    return true;
}

void fill_shapes(const uint64_t *l, int ln, const uint64_t *r, int rn) {
    fth_error_info &e = fth::last_error();
    e.lhs_ndim = ln;
    e.rhs_ndim = rn;
    for (int i = 0; i < ln && i < FTH_MAX_DIMS; ++i) e.lhs_shape[i] = l[i];
    for (int i = 0; i < rn && i < FTH_MAX_DIMS; ++i) e.rhs_shape[i] = r[i];
}

int32_t err_shape_mismatch(const fth_meta *l, const fth_meta *r) {
    set_error(FTH_ERR_SHAPE_MISMATCH, "shape mismatch: lhs rank %d, rhs rank %d", l->ndim, r->ndim);
    fill_shapes(l->shape, l->ndim, r->shape, r->ndim);
    return FTH_ERR_SHAPE_MISMATCH;
}

int32_t err_layout(const char *side) {
    set_error(FTH_ERR_UNSUPPORTED_LAYOUT, "unsupported (non-contiguous) layout on %s", side);
    std::snprintf(fth::last_error().side, sizeof(fth::last_error().side), "%s", side);
    return FTH_ERR_UNSUPPORTED_LAYOUT;
}

int32_t err_overflow(const char *context) { return set_error(FTH_ERR_SHAPE_OVERFLOW, "%s", context); }

int32_t err_invalid_dim(uint64_t dim, uint64_t ndim) {
    set_error(FTH_ERR_INVALID_DIMENSION, "invalid dimension %llu for ndim %llu", (unsigned long long)dim,
              (unsigned long long)ndim);
    fth::last_error().a = dim;
    fth::last_error().b = ndim;
    return FTH_ERR_INVALID_DIMENSION;
}

// ensure_dtype_device_and_layout[_f32] (crates/ft-kernel-cpu/src/lib.rs:2256-2284, 36935-36962):
// dtype, then device, then lhs layout, then rhs layout.
int32_t ensure_dtype_device(const fth_meta *l, const fth_meta *r) {
    if (l->dtype != r->dtype) {
        set_error(FTH_ERR_DTYPE_MISMATCH, "dtype mismatch: lhs %d, rhs %d", l->dtype, r->dtype);
        fth::last_error().a = (uint64_t)l->dtype;
        fth::last_error().b = (uint64_t)r->dtype;
        return FTH_ERR_DTYPE_MISMATCH;
    }
    if (l->device != r->device) {
        set_error(FTH_ERR_DEVICE_MISMATCH, "device mismatch: lhs %d, rhs %d", l->device, r->device);
        fth::last_error().a = (uint64_t)l->device;
        fth::last_error().b = (uint64_t)r->device;
        return FTH_ERR_DEVICE_MISMATCH;
    }
    return FTH_OK;
}
int32_t ensure_dtype_device_and_layout(const fth_meta *l, const fth_meta *r) {
    if (int32_t rc = ensure_dtype_device(l, r)) return rc;
    if (!meta_contiguous(l)) return err_layout("lhs");
    if (!meta_contiguous(r)) return err_layout("rhs");
    return FTH_OK;
}

// contiguous_required_len + ensure_storage_len (crates/ft-kernel-cpu/src/lib.rs:2340-2369).
int32_t ensure_storage_len(size_t len, const fth_meta *m, const char *side) {
    const uint64_t numel = meta_numel(m);
    uint64_t needed = 0;
    if (numel != 0 && __builtin_add_overflow(m->storage_offset, numel, &needed)) {
        set_error(FTH_ERR_STORAGE_SPAN_OVERFLOW, "storage span overflow on %s", side);
        fth_error_info &e = fth::last_error();
        std::snprintf(e.side, sizeof(e.side), "%s", side);
        e.a = m->storage_offset;
        e.b = numel;
        return FTH_ERR_STORAGE_SPAN_OVERFLOW;
    }
    if ((uint64_t)len < needed) {
        set_error(FTH_ERR_INSUFFICIENT_STORAGE, "insufficient storage on %s: needed %llu, available %llu", side,
                  (unsigned long long)needed, (unsigned long long)len);
        fth_error_info &e = fth::last_error();
        std::snprintf(e.side, sizeof(e.side), "%s", side);
        e.a = needed;
        e.b = len;
        return FTH_ERR_INSUFFICIENT_STORAGE;
    }
    return FTH_OK;
}

bool checked_mul(uint64_t a, uint64_t b, uint64_t *out) { return !__builtin_mul_overflow(a, b, out); }

// checked_dim_loop_sizes (crates/ft-kernel-cpu/src/lib.rs:2565-2574).
int32_t dim_loop_sizes(const fth_meta *m, size_t dim, const char *context, uint64_t *outer, uint64_t *inner,
                       uint64_t *total) {
    uint64_t o = 1, in = 1;
    for (size_t i = 0; i < dim; ++i)
        if (!checked_mul(o, m->shape[i], &o)) return err_overflow(context);
    for (int i = (int)dim + 1; i < m->ndim; ++i)
        if (!checked_mul(in, m->shape[i], &in)) return err_overflow(context);
    uint64_t t = 1;
    for (int i = 0; i < m->ndim; ++i)
        if (!checked_mul(t, m->shape[i], &t)) return err_overflow(context);
    *outer = o;
    *inner = in;
    *total = t;
    return FTH_OK;
}

int32_t check_out(const void *out, size_t out_cap, size_t need) {
    if (out_cap < need || (need > 0 && out == nullptr))
        return set_error(FTH_ERR_OUTPUT_TOO_SMALL, "output buffer holds %zu elements, result has %zu", out_cap, need);
    return FTH_OK;
}

// ---- staging ---------------------------------------------------------------------------------
// Small operands go over in one asynchronous copy on the library stream; anything from 1 MiB up
// goes through the pinned rings (parallel host copy overlapped with the DMA).
template <typename T> int32_t stage_in(fth::Scratch &sc, const T *host, size_t n, T **dev) {
    void *p = nullptr;
    if (int32_t rc = sc.get(&p, n * sizeof(T))) return rc;
    *dev = static_cast<T *>(p);
    if (n == 0) return FTH_OK;
    hipStream_t st = fth::resolve_stream(nullptr);
    if (n * sizeof(T) >= fth::kStagedMinBytes) return fth::staged_upload(p, host, n * sizeof(T), st);
    FTH_HIP(hipMemcpyAsync(p, host, n * sizeof(T), hipMemcpyHostToDevice, st));
    return FTH_OK;
}
template <typename T> int32_t stage_out(fth::Scratch &sc, size_t n, T **dev) {
    void *p = nullptr;
    if (int32_t rc = sc.get(&p, n * sizeof(T))) return rc;
    *dev = static_cast<T *>(p);
    return FTH_OK;
}
int32_t sync_library_stream() {
    hipError_t e = hipStreamSynchronize(fth::resolve_stream(nullptr));
    if (e != hipSuccess) {
        fth::hip_fail(e, "hipStreamSynchronize");
        fth::last_error().code = FTH_ERR_STREAM;
        return FTH_ERR_STREAM;
    }
    return FTH_OK;
}
template <typename T> int32_t fetch(T *host, const T *dev, size_t n) {
    hipStream_t st = fth::resolve_stream(nullptr);
    if (n * sizeof(T) >= fth::kStagedMinBytes) {
        if (int32_t rc = fth::staged_download(host, dev, n * sizeof(T), st)) return rc;
        return sync_library_stream();
    }
    if (n) FTH_HIP(hipMemcpyAsync(host, dev, n * sizeof(T), hipMemcpyDeviceToHost, st));
    return sync_library_stream();
}

// A row-wise op on host slices: `rows` independent rows of `cols` elements, one or two row-aligned
// inputs and a row-aligned output of the same shape. Large problems run as an upload / kernel /
// download pipeline over chunks of rows; `launch(in0, in1, out, nrows)` gets device pointers to the
// chunk. Small ones upload, launch once and download.
template <typename T, typename F>
int32_t run_rows(const T *in0, const T *in1, T *out, int64_t rows, int64_t cols, F launch) {
    const size_t total = (size_t)rows * (size_t)cols;
    fth::Scratch sc;
    fth::RowOp op;
    op.n_in = in1 ? 2 : 1;
    op.host_in[0] = in0; op.host_in[1] = in1;
    op.in_row_bytes[0] = (size_t)cols * sizeof(T);
    op.in_row_bytes[1] = in1 ? (size_t)cols * sizeof(T) : 0;
    op.host_out = out;
    op.out_row_bytes = (size_t)cols * sizeof(T);
    op.rows = rows;
    if (!fth::row_pipeline_applies(op)) {
        T *d0, *d1 = nullptr, *dy;
        if (int32_t rc = stage_in(sc, in0, total, &d0)) return rc;
        if (in1)
            if (int32_t rc = stage_in(sc, in1, total, &d1)) return rc;
        if (int32_t rc = stage_out(sc, total, &dy)) return rc;
        if (int32_t rc = launch(d0, d1, dy, rows)) return rc;
        return fetch(out, dy, total);
    }
    T *d0, *d1 = nullptr, *dy;
    if (int32_t rc = stage_out(sc, total, &d0)) return rc;
    if (in1)
        if (int32_t rc = stage_out(sc, total, &d1)) return rc;
    if (int32_t rc = stage_out(sc, total, &dy)) return rc;
    op.dev_in[0] = d0; op.dev_in[1] = d1; op.dev_out = dy;
    if (int32_t rc = fth::row_pipeline(op, [&](int64_t row0, int64_t nrows) {
            return launch(d0 + row0 * cols, d1 ? d1 + row0 * cols : nullptr, dy + row0 * cols, nrows);
        }, fth::resolve_stream(nullptr)))
        return rc;
    return sync_library_stream();
}

template <typename T> struct Dev;
template <> struct Dev<float> {
    static int32_t gemm(const fth_gemm_desc *d, float al, const float *a, const float *b, float *c, const float *bias) {
        return fth_dev_gemm_f32(d, al, a, b, c, bias, nullptr, nullptr);
    }
    static int32_t softmax(const float *x, float *y, int64_t o, int64_t r, int64_t i) { return fth_dev_softmax_strided_f32(x, y, o, r, i, nullptr); }
    static int32_t sdpa_masked(const fth_sdpa_desc *d, float sc, const float *q, const float *k, const float *v, const float *m, int64_t ms, float *o) {
        return fth_dev_sdpa_forward_masked_f32(d, sc, q, k, v, m, ms, o, nullptr);
    }
    static int32_t log_softmax(const float *x, float *y, int64_t o, int64_t r, int64_t i) { return fth_dev_log_softmax_strided_f32(x, y, o, r, i, nullptr); }
    static int32_t ce_fwd(const float *l, const int64_t *t, int64_t b, int64_t c, float *o, int64_t *bad) { return fth_dev_cross_entropy_forward_f32(l, t, b, c, o, bad, nullptr); }
    static int32_t ce_bwd(const float *l, const int64_t *t, const float *g, int64_t b, int64_t c, float *o, int64_t *bad) { return fth_dev_cross_entropy_backward_f32(l, t, g, b, c, o, bad, nullptr); }
    static int32_t layer_norm(const float *x, const float *w, const float *b, float *y, int64_t n, int64_t c, float e) { return fth_dev_layer_norm_f32(x, w, b, y, n, c, e, nullptr); }
    static int32_t rms_norm(const float *x, const float *w, float *y, int64_t n, int64_t c, float e) { return fth_dev_rms_norm_f32(x, w, y, n, c, e, nullptr); }
    static int32_t gelu(const float *x, float *y, int64_t n) { return fth_dev_gelu_f32(x, y, n, nullptr); }
    static int32_t gelu_tanh(const float *x, float *y, int64_t n) { return fth_dev_gelu_tanh_f32(x, y, n, nullptr); }
    static int32_t add(const float *a, const float *b, float *y, int64_t n) { return fth_dev_add_f32(a, b, y, n, nullptr); }
    static int32_t sdpa(const fth_sdpa_desc *d, float s, const float *q, const float *k, const float *v, float *o) { return fth_dev_sdpa_forward_f32(d, s, q, k, v, o, nullptr); }
    static int32_t index_select(const float *x, int64_t o, int64_t ds, int64_t in, const double *idx, int64_t n, float *out) { return fth_dev_index_select_f32(x, o, ds, in, idx, n, out, nullptr, nullptr); }
    static int32_t argmax(const float *x, int64_t o, int64_t r, int64_t in, float *out) { return fth_dev_argmax_f32(x, o, r, in, out, nullptr); }
    static constexpr int32_t dtype = FTH_DTYPE_F32;
};
template <> struct Dev<double> {
    static int32_t gemm(const fth_gemm_desc *d, double al, const double *a, const double *b, double *c, const double *bias) {
        return fth_dev_gemm_f64(d, al, a, b, c, bias, nullptr, nullptr);
    }
    static int32_t softmax(const double *x, double *y, int64_t o, int64_t r, int64_t i) { return fth_dev_softmax_strided_f64(x, y, o, r, i, nullptr); }
    static int32_t sdpa_masked(const fth_sdpa_desc *d, double sc, const double *q, const double *k, const double *v, const double *m, int64_t ms, double *o) {
        return fth_dev_sdpa_forward_masked_f64(d, sc, q, k, v, m, ms, o, nullptr);
    }
    static int32_t log_softmax(const double *x, double *y, int64_t o, int64_t r, int64_t i) { return fth_dev_log_softmax_strided_f64(x, y, o, r, i, nullptr); }
    static int32_t ce_fwd(const double *l, const int64_t *t, int64_t b, int64_t c, double *o, int64_t *bad) { return fth_dev_cross_entropy_forward_f64(l, t, b, c, o, bad, nullptr); }
    static int32_t ce_bwd(const double *l, const int64_t *t, const double *g, int64_t b, int64_t c, double *o, int64_t *bad) { return fth_dev_cross_entropy_backward_f64(l, t, g, b, c, o, bad, nullptr); }
    static int32_t layer_norm(const double *x, const double *w, const double *b, double *y, int64_t n, int64_t c, double e) { return fth_dev_layer_norm_f64(x, w, b, y, n, c, e, nullptr); }
    static int32_t rms_norm(const double *x, const double *w, double *y, int64_t n, int64_t c, double e) { return fth_dev_rms_norm_f64(x, w, y, n, c, e, nullptr); }
    static int32_t gelu(const double *x, double *y, int64_t n) { return fth_dev_gelu_f64(x, y, n, nullptr); }
    static int32_t gelu_tanh(const double *x, double *y, int64_t n) { return fth_dev_gelu_tanh_f64(x, y, n, nullptr); }
    static int32_t add(const double *a, const double *b, double *y, int64_t n) { return fth_dev_add_f64(a, b, y, n, nullptr); }
    static int32_t sdpa(const fth_sdpa_desc *d, double s, const double *q, const double *k, const double *v, double *o) { return fth_dev_sdpa_forward_f64(d, s, q, k, v, o, nullptr); }
    static int32_t index_select(const double *x, int64_t o, int64_t ds, int64_t in, const double *idx, int64_t n, double *out) { return fth_dev_index_select_f64(x, o, ds, in, idx, n, out, nullptr, nullptr); }
    static int32_t argmax(const double *x, int64_t o, int64_t r, int64_t in, double *out) { return fth_dev_argmax_f64(x, o, r, in, out, nullptr); }
    static constexpr int32_t dtype = FTH_DTYPE_F64;
};

fth_gemm_desc gemm_desc(int64_t m, int64_t n, int64_t k, int trans_b, int64_t batch, int epi) {
    fth_gemm_desc d{};
    d.m = m; d.n = n; d.k = k;
    d.lda = k; d.ldb = trans_b ? k : n; d.ldc = n;
    d.batch = batch;
    d.stride_a = m * k; d.stride_b = k * n; d.stride_c = m * n;
    d.trans_b = trans_b;
    d.epilogue = epi;
    return d;
}

// The addmm combine of crates/ft-kernel-cpu/src/lib.rs:41614-41645: two multiplies, one add.
template <typename T>
__global__ __launch_bounds__(256) void addmm_combine_kernel(const T *__restrict__ input, int input_1d,
                                                            const T *__restrict__ g, T *__restrict__ out,
                                                            int64_t total, int64_t n, T beta, T alpha, int alpha_zero) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const T in = input_1d ? input[i % n] : input[i];
    out[i] = alpha_zero ? beta * in : beta * in + alpha * g[i];
}

// ---- matmul_tensor_contiguous (crates/ft-kernel-cpu/src/lib.rs:37780-37823 / 17355-17379) ------
template <typename T>
int32_t matmul_impl(const T *lhs, size_t lhs_len, const T *rhs, size_t rhs_len, const fth_meta *lm, const fth_meta *rm,
                    T *out, size_t out_cap, size_t *out_len) {
    FTH_ARG(meta_ok(lm) && meta_ok(rm), "matmul: bad meta");
    if (out_len) *out_len = 0;
    if (int32_t rc = ensure_dtype_device_and_layout(lm, rm)) return rc;
    if (lm->ndim != 2 || rm->ndim != 2 || lm->shape[1] != rm->shape[0]) return err_shape_mismatch(lm, rm);
    const uint64_t m = lm->shape[0], k = lm->shape[1], n = rm->shape[1];
    uint64_t t, out_numel;
    if (!checked_mul(m, k, &t)) return err_overflow("matmul lhs overflow");
    if (!checked_mul(k, n, &t)) return err_overflow("matmul rhs overflow");
    if (!checked_mul(m, n, &out_numel)) return err_overflow("matmul output overflow");
    if (int32_t rc = ensure_storage_len(lhs_len, lm, "lhs")) return rc;
    if (int32_t rc = ensure_storage_len(rhs_len, rm, "rhs")) return rc;
    if (out_len) *out_len = (size_t)out_numel;
    if (out == nullptr && out_cap == 0) return FTH_OK;  // validation only
    if (int32_t rc = check_out(out, out_cap, (size_t)out_numel)) return rc;
    if (out_numel == 0) return FTH_OK;
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    T *da, *db, *dc;
    if (int32_t rc = stage_in(sc, lhs + lm->storage_offset, (size_t)(m * k), &da)) return rc;
    if (int32_t rc = stage_in(sc, rhs + rm->storage_offset, (size_t)(k * n), &db)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)out_numel, &dc)) return rc;
    fth_gemm_desc d = gemm_desc((int64_t)m, (int64_t)n, (int64_t)k, 0, 1, FTH_EPI_NONE);
    if (int32_t rc = Dev<T>::gemm(&d, T(1), da, db, dc, nullptr)) return rc;
    return fetch(out, dc, (size_t)out_numel);
}

// ---- bmm_tensor_contiguous (crates/ft-kernel-cpu/src/lib.rs:38496-38606 / 17785-17872) --------
template <typename T>
int32_t bmm_impl(const T *lhs, size_t lhs_len, const T *rhs, size_t rhs_len, const fth_meta *lm, const fth_meta *rm,
                 T *out, size_t out_cap, size_t *out_len) {
    FTH_ARG(meta_ok(lm) && meta_ok(rm), "bmm: bad meta");
    if (out_len) *out_len = 0;
    if (int32_t rc = ensure_dtype_device_and_layout(lm, rm)) return rc;
    if (lm->ndim != 3 || rm->ndim != 3) return err_shape_mismatch(lm, rm);
    const uint64_t batch = lm->shape[0], m = lm->shape[1], k = lm->shape[2], n = rm->shape[2];
    if (batch != rm->shape[0] || k != rm->shape[1]) return err_shape_mismatch(lm, rm);
    uint64_t ls, rs, os, t, out_numel;
    if (!checked_mul(m, k, &ls)) return err_overflow("bmm lhs batch stride overflow");
    if (!checked_mul(k, n, &rs)) return err_overflow("bmm rhs batch stride overflow");
    if (!checked_mul(m, n, &os)) return err_overflow("bmm output batch stride overflow");
    if (!checked_mul(batch, ls, &t)) return err_overflow("bmm lhs overflow");
    if (!checked_mul(batch, rs, &t)) return err_overflow("bmm rhs overflow");
    if (!checked_mul(batch, os, &out_numel)) return err_overflow("bmm output overflow");
    if (int32_t rc = ensure_storage_len(lhs_len, lm, "lhs")) return rc;
    if (int32_t rc = ensure_storage_len(rhs_len, rm, "rhs")) return rc;
    if (out_len) *out_len = (size_t)out_numel;
    if (out == nullptr && out_cap == 0) return FTH_OK;
    if (int32_t rc = check_out(out, out_cap, (size_t)out_numel)) return rc;
    if (out_numel == 0) return FTH_OK;
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    T *da, *db, *dc;
    if (int32_t rc = stage_in(sc, lhs + lm->storage_offset, (size_t)(batch * ls), &da)) return rc;
    if (int32_t rc = stage_in(sc, rhs + rm->storage_offset, (size_t)(batch * rs), &db)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)out_numel, &dc)) return rc;
    // The grid's batch axis holds 65 535 entries; larger batches go in slices.
    for (uint64_t b0 = 0; b0 < batch; b0 += 65535) {
        const uint64_t nb = (batch - b0) < 65535 ? (batch - b0) : 65535;
        fth_gemm_desc d = gemm_desc((int64_t)m, (int64_t)n, (int64_t)k, 0, (int64_t)nb, FTH_EPI_NONE);
        if (int32_t rc = Dev<T>::gemm(&d, T(1), da + b0 * ls, db + b0 * rs, dc + b0 * os, nullptr)) return rc;
    }
    return fetch(out, dc, (size_t)out_numel);
}

// ---- addmm_tensor_contiguous (crates/ft-kernel-cpu/src/lib.rs:41562-41648 / 17514-17606) ------
template <typename T>
int32_t addmm_impl(const T *input, size_t input_len, const T *mat1, size_t mat1_len, const T *mat2, size_t mat2_len,
                   const fth_meta *im, const fth_meta *m1, const fth_meta *m2, T beta, T alpha, T *out,
                   size_t out_cap, size_t *out_len) {
    FTH_ARG(meta_ok(im) && meta_ok(m1) && meta_ok(m2), "addmm: bad meta");
    if (out_len) *out_len = 0;
    if (m1->ndim != 2 || m2->ndim != 2 || m1->shape[1] != m2->shape[0]) return err_shape_mismatch(m1, m2);
    const uint64_t m = m1->shape[0], k = m1->shape[1], n = m2->shape[1];
    uint64_t out_numel;
    if (!checked_mul(m, n, &out_numel)) return err_overflow("addmm output overflow");
    if (int32_t rc = ensure_storage_len(mat1_len, m1, "mat1")) return rc;
    if (int32_t rc = ensure_storage_len(mat2_len, m2, "mat2")) return rc;
    const bool in1d = im->ndim == 1 && im->shape[0] == n;
    const bool in2d = im->ndim == 2 && im->shape[0] == m && im->shape[1] == n;
    if (!in1d && !in2d) {
        set_error(FTH_ERR_SHAPE_MISMATCH, "addmm: input shape does not broadcast to [m, n]");
        const uint64_t want[2] = {m, n};
        fill_shapes(im->shape, im->ndim, want, 2);
        return FTH_ERR_SHAPE_MISMATCH;
    }
    if (int32_t rc = ensure_storage_len(input_len, im, "input")) return rc;
    if (!meta_contiguous(m1)) return err_layout("mat1");
    if (!meta_contiguous(m2)) return err_layout("mat2");
    if (!meta_contiguous(im)) return err_layout("input");
    if (out_len) *out_len = (size_t)out_numel;
    if (out == nullptr && out_cap == 0) return FTH_OK;
    if (int32_t rc = check_out(out, out_cap, (size_t)out_numel)) return rc;
    if (out_numel == 0) return FTH_OK;
    FTH_REQUIRE_DEVICE();
    // alpha.to_bits() == 0: only +0.0 takes the shortcut (crates/ft-kernel-cpu/src/lib.rs:41614).
    bool alpha_zero;
    if constexpr (sizeof(T) == 4) {
        uint32_t bits;
        std::memcpy(&bits, &alpha, 4);
        alpha_zero = bits == 0;
    } else {
        uint64_t bits;
        std::memcpy(&bits, &alpha, 8);
        alpha_zero = bits == 0;
    }
    fth::Scratch sc;
    T *di, *d1 = nullptr, *d2 = nullptr, *dg = nullptr, *dout;
    if (int32_t rc = stage_in(sc, input + im->storage_offset, (size_t)(in1d ? n : out_numel), &di)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)out_numel, &dout)) return rc;
    if (!alpha_zero) {
        if (int32_t rc = stage_in(sc, mat1 + m1->storage_offset, (size_t)(m * k), &d1)) return rc;
        if (int32_t rc = stage_in(sc, mat2 + m2->storage_offset, (size_t)(k * n), &d2)) return rc;
        if (int32_t rc = stage_out(sc, (size_t)out_numel, &dg)) return rc;
        fth_gemm_desc d = gemm_desc((int64_t)m, (int64_t)n, (int64_t)k, 0, 1, FTH_EPI_NONE);
        if (int32_t rc = Dev<T>::gemm(&d, T(1), d1, d2, dg, nullptr)) return rc;
    }
    const int64_t grid = fth::ceil_div((int64_t)out_numel, 256);
    FTH_ARG(grid <= 2147483647LL, "addmm: output too large for one launch");
    addmm_combine_kernel<T><<<dim3((unsigned)grid), dim3(256), 0, fth::resolve_stream(nullptr)>>>(
        di, in1d ? 1 : 0, dg, dout, (int64_t)out_numel, (int64_t)n, beta, alpha, alpha_zero ? 1 : 0);
    FTH_CHECK_LAUNCH("addmm_combine");
    return fetch(out, dout, (size_t)out_numel);
}

// ---- linear_tensor (crates/ft-kernel-cpu/src/lib.rs:17306-17353 / 17162-17211) ----------------
// The reference is infallible and panics on short slices; here that is FTH_ERR_INVALID_ARGUMENT.
template <typename T>
int32_t linear_impl(const T *x, size_t x_len, const T *w, size_t w_len, const T *bias, size_t bias_len, size_t batch,
                    size_t in_f, size_t out_f, T *out, size_t out_cap, size_t *out_len) {
    uint64_t xn, wn, on;
    FTH_ARG(checked_mul(batch, in_f, &xn) && checked_mul(out_f, in_f, &wn) && checked_mul(batch, out_f, &on),
            "linear: shape product overflows");
    if (out_len) *out_len = (size_t)on;
    if (out == nullptr && out_cap == 0) return FTH_OK;
    if (int32_t rc = check_out(out, out_cap, (size_t)on)) return rc;
    if (on == 0) return FTH_OK;
    FTH_ARG(x_len >= xn && w_len >= wn, "linear: slice shorter than batch*in (%zu < %llu) or out*in (%zu < %llu)", x_len,
            (unsigned long long)xn, w_len, (unsigned long long)wn);
    FTH_ARG(bias == nullptr || bias_len >= out_f, "linear: bias shorter than out_features");
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    T *dx, *dw, *db = nullptr, *dy;
    if (int32_t rc = stage_in(sc, x, (size_t)xn, &dx)) return rc;
    if (int32_t rc = stage_in(sc, w, (size_t)wn, &dw)) return rc;
    if (bias)
        if (int32_t rc = stage_in(sc, bias, out_f, &db)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)on, &dy)) return rc;
    fth_gemm_desc d = gemm_desc((int64_t)batch, (int64_t)out_f, (int64_t)in_f, 1, 1, bias ? FTH_EPI_BIAS : FTH_EPI_NONE);
    if (int32_t rc = Dev<T>::gemm(&d, T(1), dx, dw, dy, db)) return rc;
    return fetch(out, dy, (size_t)on);
}

// ---- matmul_rhs_transposed_contiguous (crates/ft-kernel-cpu/src/lib.rs:17381-17436) -----------
template <typename T>
int32_t matmul_bt_impl(size_t m, size_t k, size_t n, const T *lhs, size_t lhs_len, const T *rhs, size_t rhs_len, T *out,
                       size_t out_cap, size_t *out_len) {
    if (out_len) *out_len = 0;
    uint64_t ll, rl, ol;
    if (!checked_mul(m, k, &ll)) return err_overflow("matmul_rhs_transposed lhs overflow");
    if (!checked_mul(n, k, &rl)) return err_overflow("matmul_rhs_transposed rhs overflow");
    if (!checked_mul(m, n, &ol)) return err_overflow("matmul_rhs_transposed output overflow");
    if (lhs_len < ll) {
        set_error(FTH_ERR_SHAPE_MISMATCH, "matmul_rhs_transposed: lhs slice shorter than m*k");
        const uint64_t a[1] = {ll}, b[1] = {lhs_len};
        fill_shapes(a, 1, b, 1);
        return FTH_ERR_SHAPE_MISMATCH;
    }
    if (rhs_len < rl) {
        set_error(FTH_ERR_SHAPE_MISMATCH, "matmul_rhs_transposed: rhs slice shorter than n*k");
        const uint64_t a[1] = {rl}, b[1] = {rhs_len};
        fill_shapes(a, 1, b, 1);
        return FTH_ERR_SHAPE_MISMATCH;
    }
    if (out_len) *out_len = (size_t)ol;
    if (out == nullptr && out_cap == 0) return FTH_OK;
    if (int32_t rc = check_out(out, out_cap, (size_t)ol)) return rc;
    if (ol == 0) return FTH_OK;
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    T *da, *db, *dc;
    if (int32_t rc = stage_in(sc, lhs, (size_t)ll, &da)) return rc;
    if (int32_t rc = stage_in(sc, rhs, (size_t)rl, &db)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)ol, &dc)) return rc;
    fth_gemm_desc d = gemm_desc((int64_t)m, (int64_t)n, (int64_t)k, 1, 1, FTH_EPI_NONE);
    if (int32_t rc = Dev<T>::gemm(&d, T(1), da, db, dc, nullptr)) return rc;
    return fetch(out, dc, (size_t)ol);
}

// ---- unary / dim ops -----------------------------------------------------------------------
int32_t ensure_unary(size_t len, const fth_meta *m) {
    if (!meta_contiguous(m)) return err_layout("input");
    return ensure_storage_len(len, m, "input");
}

// softmax_dim_tensor_contiguous (crates/ft-kernel-cpu/src/lib.rs:39193-39296 / 18350-18461)
template <typename T>
int32_t softmax_impl(const T *input, size_t input_len, const fth_meta *meta, size_t dim, T *out, size_t out_cap,
                     size_t *out_len, bool log_form = false) {
    FTH_ARG(meta_ok(meta), "softmax: bad meta");
    if (out_len) *out_len = 0;
    if (int32_t rc = ensure_unary(input_len, meta)) return rc;
    if (dim >= (size_t)meta->ndim) return err_invalid_dim(dim, (uint64_t)meta->ndim);
    uint64_t outer, inner, numel;
    if (int32_t rc = dim_loop_sizes(meta, dim, "softmax overflow", &outer, &inner, &numel)) return rc;
    if (out_len) *out_len = (size_t)numel;
    if (out == nullptr && out_cap == 0) return FTH_OK;
    if (int32_t rc = check_out(out, out_cap, (size_t)numel)) return rc;
    if (numel == 0) return FTH_OK;
    FTH_REQUIRE_DEVICE();
    // log_softmax_dim_tensor_contiguous (crates/ft-kernel-cpu/src/lib.rs:39298-39375 / 18504-18590) shares the validation
    const int64_t reduce = (int64_t)meta->shape[dim];
    if (inner == 1 && outer <= (uint64_t)std::numeric_limits<int64_t>::max()) {
        // last-dim form: the rows are independent, so transfers and kernels overlap chunk by chunk
        return run_rows<T>(input + meta->storage_offset, nullptr, out, (int64_t)outer, reduce, [&](const T *x, const T *, T *y, int64_t nrows) {
            return log_form ? Dev<T>::log_softmax(x, y, nrows, reduce, 1) : Dev<T>::softmax(x, y, nrows, reduce, 1);
        });
    }
    fth::Scratch sc;
    T *dx, *dy;
    if (int32_t rc = stage_in(sc, input + meta->storage_offset, (size_t)numel, &dx)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)numel, &dy)) return rc;
    if (int32_t rc = log_form ? Dev<T>::log_softmax(dx, dy, (int64_t)outer, reduce, (int64_t)inner)
                              : Dev<T>::softmax(dx, dy, (int64_t)outer, reduce, (int64_t)inner))
        return rc;
    return fetch(out, dy, (size_t)numel);
}

// layer_norm_forward (crates/ft-kernel-cpu/src/lib.rs:5877-5923 / 5824-5870), optionally fused
// with the residual add (add_layer_norm_forward_f32, :5932-5984).
template <typename T>
int32_t layer_norm_impl(const T *x, const T *x2, size_t x_len, const T *w, const T *b, size_t batch, size_t n, T eps,
                        T *out, size_t out_cap) {
    uint64_t total;
    FTH_ARG(checked_mul(batch, n, &total), "layer_norm: batch * norm_size overflows");
    if (int32_t rc = check_out(out, out_cap, (size_t)total)) return rc;
    if (total == 0) return FTH_OK;
    FTH_ARG(x_len >= total, "layer_norm: input slice shorter than batch * norm_size");
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    T *dw = nullptr, *db = nullptr;
    if (w)
        if (int32_t rc = stage_in(sc, w, n, &dw)) return rc;
    if (b)
        if (int32_t rc = stage_in(sc, b, n, &db)) return rc;
    return run_rows<T>(x, x2, out, (int64_t)batch, (int64_t)n, [&](const T *dx, const T *dx2, T *dy, int64_t nrows) -> int32_t {
        if constexpr (std::is_same<T, float>::value) {
            return dx2 ? fth_dev_add_layer_norm_f32(dx, dx2, dw, db, dy, nrows, (int64_t)n, eps, nullptr)
                       : fth_dev_layer_norm_f32(dx, dw, db, dy, nrows, (int64_t)n, eps, nullptr);
        } else {
            return fth_dev_layer_norm_f64(dx, dw, db, dy, nrows, (int64_t)n, eps, nullptr);
        }
    });
}

// rms_norm_forward (crates/ft-kernel-cpu/src/lib.rs:6459-6494 / 6418-6453)
template <typename T>
int32_t rms_norm_impl(const T *x, size_t x_len, const T *w, size_t batch, size_t n, T eps, T *out, size_t out_cap) {
    uint64_t total;
    FTH_ARG(checked_mul(batch, n, &total), "rms_norm: batch * norm_size overflows");
    if (int32_t rc = check_out(out, out_cap, (size_t)total)) return rc;
    if (total == 0) return FTH_OK;
    FTH_ARG(x_len >= total, "rms_norm: input slice shorter than batch * norm_size");
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    T *dw = nullptr;
    if (w)
        if (int32_t rc = stage_in(sc, w, n, &dw)) return rc;
    return run_rows<T>(x, nullptr, out, (int64_t)batch, (int64_t)n, [&](const T *dx, const T *, T *dy, int64_t nrows) {
        return Dev<T>::rms_norm(dx, dw, dy, nrows, (int64_t)n, eps);
    });
}

// gelu_tensor_contiguous (unary_contiguous_f32 via define_unary_f32!, crates/ft-kernel-cpu/src/
// lib.rs:37051-37064, 37123-37127)
template <typename T>
int32_t gelu_impl(const T *input, size_t input_len, const fth_meta *meta, T *out, size_t out_cap, size_t *out_len, bool tanh_form = false) {
    FTH_ARG(meta_ok(meta), "gelu: bad meta");
    if (out_len) *out_len = 0;
    if (int32_t rc = ensure_unary(input_len, meta)) return rc;
    const uint64_t numel = meta_numel(meta);
    if (out_len) *out_len = (size_t)numel;
    if (out == nullptr && out_cap == 0) return FTH_OK;
    if (int32_t rc = check_out(out, out_cap, (size_t)numel)) return rc;
    if (numel == 0) return FTH_OK;
    FTH_REQUIRE_DEVICE();
    // elementwise: every element is a "row" of its own, so the pipeline cuts the tensor anywhere
    FTH_ARG(numel <= (uint64_t)std::numeric_limits<int64_t>::max(), "gelu: tensor too large");
    return run_rows<T>(input + meta->storage_offset, nullptr, out, (int64_t)numel, 1, [&](const T *dx, const T *, T *dy, int64_t count) {
        return tanh_form ? Dev<T>::gelu_tanh(dx, dy, count) : Dev<T>::gelu(dx, dy, count);
    });
}

// add_tensor_contiguous (simd_elementwise_f32, crates/ft-kernel-cpu/src/lib.rs:36558-36593):
// dtype, device, equal shapes, then storage lengths; no broadcast.
template <typename T>
int32_t add_impl(const T *lhs, size_t lhs_len, const T *rhs, size_t rhs_len, const fth_meta *lm, const fth_meta *rm,
                 T *out, size_t out_cap, size_t *out_len) {
    FTH_ARG(meta_ok(lm) && meta_ok(rm), "add: bad meta");
    if (out_len) *out_len = 0;
    if (int32_t rc = ensure_dtype_device(lm, rm)) return rc;
    bool same = lm->ndim == rm->ndim;
    for (int i = 0; same && i < lm->ndim; ++i) same = lm->shape[i] == rm->shape[i];
    if (!same) return err_shape_mismatch(lm, rm);
    if (int32_t rc = ensure_storage_len(lhs_len, lm, "lhs")) return rc;
    if (int32_t rc = ensure_storage_len(rhs_len, rm, "rhs")) return rc;
    const uint64_t numel = meta_numel(lm);
    if (out_len) *out_len = (size_t)numel;
    if (out == nullptr && out_cap == 0) return FTH_OK;
    if (int32_t rc = check_out(out, out_cap, (size_t)numel)) return rc;
    if (numel == 0) return FTH_OK;
    FTH_REQUIRE_DEVICE();
    FTH_ARG(numel <= (uint64_t)std::numeric_limits<int64_t>::max(), "add: tensor too large");
    return run_rows<T>(lhs + lm->storage_offset, rhs + rm->storage_offset, out, (int64_t)numel, 1, [&](const T *da, const T *db, T *dy, int64_t count) {
        return Dev<T>::add(da, db, dy, count);
    });
}

// sdpa_forward (crates/ft-kernel-cpu/src/lib.rs:5200-5284 / 4572-4651)
template <typename T>
int32_t sdpa_impl(const T *q, size_t q_len, const T *k, size_t k_len, const T *v, size_t v_len, size_t num_bh,
                  size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, T scale, int32_t causal, T *out, size_t out_cap) {
    uint64_t qn, kn, vn, on, t;
    FTH_ARG(checked_mul(num_bh, seq_q, &t) && checked_mul(t, d_k, &qn) && checked_mul(t, d_v, &on) &&
                checked_mul(num_bh, seq_k, &t) && checked_mul(t, d_k, &kn) && checked_mul(t, d_v, &vn),
            "sdpa: shape product overflows");
    if (int32_t rc = check_out(out, out_cap, (size_t)on)) return rc;
    if (on == 0) return FTH_OK;
    FTH_ARG(q_len >= qn && k_len >= kn && v_len >= vn, "sdpa: q/k/v slice shorter than its shape");
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    T *dq, *dk, *dv, *dout;
    if (int32_t rc = stage_in(sc, q, (size_t)qn, &dq)) return rc;
    if (int32_t rc = stage_in(sc, k, (size_t)kn, &dk)) return rc;
    if (int32_t rc = stage_in(sc, v, (size_t)vn, &dv)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)on, &dout)) return rc;
    fth_sdpa_desc d;
    fth_sdpa_desc_contiguous(&d, (int64_t)num_bh, (int64_t)seq_q, (int64_t)seq_k, (int64_t)d_k, (int64_t)d_v, causal ? 1 : 0);
    if (int32_t rc = Dev<T>::sdpa(&d, scale, dq, dk, dv, dout)) return rc;
    return fetch(out, dout, (size_t)on);
}

// sdpa_forward_masked_gqa_f64 (crates/ft-kernel-cpu/src/lib.rs:4777-4850) and, with h_q == h_kv, sdpa_forward_masked_f64
// (:4661-4741): q [batch, h_q, seq_q, d_k], k / v [batch, h_kv, seq_k, d], additive mask with mask_bh_stride 0 (shared
// [seq_q, seq_k]) or seq_q * seq_k (one per batch * h_q). The reference indexes the mask slice and panics when it is
// short; that is InvalidArgument here.
template <typename T>
int32_t sdpa_masked_impl(const T *q, size_t q_len, const T *k, size_t k_len, const T *v, size_t v_len, size_t batch, size_t h_q,
                         size_t h_kv, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, T scale, const T *mask, size_t mask_len,
                         size_t mask_bh_stride, T *out, size_t out_cap) {
    FTH_ARG(h_kv > 0 && h_q % h_kv == 0, "sdpa_masked_gqa: h_kv (%zu) must divide h_q (%zu)", h_kv, h_q);
    uint64_t num_bh, num_kv, qn, kn, vn, on, mn, t;
    FTH_ARG(checked_mul(batch, h_q, &num_bh) && checked_mul(batch, h_kv, &num_kv) && checked_mul(num_bh, seq_q, &t) &&
                checked_mul(t, d_k, &qn) && checked_mul(t, d_v, &on) && checked_mul(num_kv, seq_k, &t) && checked_mul(t, d_k, &kn) &&
                checked_mul(t, d_v, &vn) && checked_mul(seq_q, seq_k, &mn),
            "sdpa_masked: shape product overflows");
    if (int32_t rc = check_out(out, out_cap, (size_t)on)) return rc;
    if (on == 0) return FTH_OK;
    FTH_ARG(q_len >= qn && k_len >= kn && v_len >= vn, "sdpa_masked: q/k/v slice shorter than its shape");
    FTH_ARG(mask_bh_stride == 0 || mask_bh_stride >= mn, "sdpa_masked: mask_bh_stride %zu is neither 0 nor >= seq_q * seq_k", mask_bh_stride);
    uint64_t mask_need;
    FTH_ARG(checked_mul(num_bh - 1, mask_bh_stride, &mask_need) && !__builtin_add_overflow(mask_need, mn, &mask_need) && mask_len >= mask_need,
            "sdpa_masked: mask slice (%zu) shorter than the %llu elements the shape reads", mask_len, (unsigned long long)mask_need);
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    T *dq, *dk, *dv, *dm = nullptr, *dout;
    if (int32_t rc = stage_in(sc, q, (size_t)qn, &dq)) return rc;
    if (int32_t rc = stage_in(sc, k, (size_t)kn, &dk)) return rc;
    if (int32_t rc = stage_in(sc, v, (size_t)vn, &dv)) return rc;
    if (mask_need > 0)
        if (int32_t rc = stage_in(sc, mask, (size_t)mask_need, &dm)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)on, &dout)) return rc;
    fth_sdpa_desc d;
    fth_sdpa_desc_contiguous(&d, (int64_t)num_bh, (int64_t)seq_q, (int64_t)seq_k, (int64_t)d_k, (int64_t)d_v, 0);
    d.heads = (int64_t)h_q;
    d.kv_group = (int32_t)(h_q / h_kv);
    FTH_ARG(h_q / h_kv <= 2147483647ull, "sdpa_masked_gqa: group too large");
    d.q_batch_stride = (int64_t)(h_q * seq_q * d_k); d.q_head_stride = (int64_t)(seq_q * d_k);
    d.k_batch_stride = (int64_t)(h_kv * seq_k * d_k); d.k_head_stride = (int64_t)(seq_k * d_k);
    d.v_batch_stride = (int64_t)(h_kv * seq_k * d_v); d.v_head_stride = (int64_t)(seq_k * d_v);
    d.o_batch_stride = (int64_t)(h_q * seq_q * d_v); d.o_head_stride = (int64_t)(seq_q * d_v);
    if (int32_t rc = Dev<T>::sdpa_masked(&d, scale, dq, dk, dv, dm, (int64_t)mask_bh_stride, dout)) return rc;
    return fetch(out, dout, (size_t)on);
}

// normalize_strict_index_value (crates/ft-kernel-cpu/src/lib.rs:20058-20090), host side: the
// reference returns Err at the first bad index before producing anything.
bool strict_index_ok(double v, uint64_t dim_size) {
    if (!std::isfinite(v)) return false;
    if (std::fabs(v - std::trunc(v)) > std::numeric_limits<double>::epsilon()) return false;
    if (v < 0.0 || v >= 9.2233720368547758e18) return false;
    return (uint64_t)(int64_t)v < dim_size;
}

// index_select_tensor_contiguous (crates/ft-kernel-cpu/src/lib.rs:40216-40253)
template <typename T>
int32_t index_select_impl(const T *input, size_t input_len, const fth_meta *meta, size_t dim, const double *indices,
                          size_t num_indices, T *out, size_t out_cap, size_t *out_len) {
    FTH_ARG(meta_ok(meta), "index_select: bad meta");
    if (out_len) *out_len = 0;
    if (int32_t rc = ensure_unary(input_len, meta)) return rc;
    if (dim >= (size_t)meta->ndim) return err_invalid_dim(dim, (uint64_t)meta->ndim);
    const uint64_t dim_size = meta->shape[dim];
    uint64_t outer, inner, total, t, out_numel;
    if (int32_t rc = dim_loop_sizes(meta, dim, "index_select overflow", &outer, &inner, &total)) return rc;
    if (!checked_mul(outer, num_indices, &t) || !checked_mul(t, inner, &out_numel)) return err_overflow("index_select overflow");
    if (out_numel == 0) return FTH_OK;  // empty result before any index is looked at, as in the reference
    FTH_ARG(indices != nullptr, "index_select: indices is NULL");
    for (size_t i = 0; i < num_indices; ++i)
        if (!strict_index_ok(indices[i], dim_size)) return err_invalid_dim(dim_size, dim_size);
    if (out_len) *out_len = (size_t)out_numel;
    if (out == nullptr && out_cap == 0) return FTH_OK;
    if (int32_t rc = check_out(out, out_cap, (size_t)out_numel)) return rc;
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    T *dx, *dy;
    double *di;
    if (int32_t rc = stage_in(sc, input + meta->storage_offset, (size_t)total, &dx)) return rc;
    if (int32_t rc = stage_in(sc, indices, num_indices, &di)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)out_numel, &dy)) return rc;
    if (int32_t rc = Dev<T>::index_select(dx, (int64_t)outer, (int64_t)dim_size, (int64_t)inner, di, (int64_t)num_indices, dy)) return rc;
    return fetch(out, dy, (size_t)out_numel);
}

// argmax_dim_tensor_contiguous (crates/ft-kernel-cpu/src/lib.rs:39443-39550 / 18653)
template <typename T>
int32_t argmax_impl(const T *input, size_t input_len, const fth_meta *meta, size_t dim, T *out, size_t out_cap,
                    size_t *out_len) {
    FTH_ARG(meta_ok(meta), "argmax: bad meta");
    if (out_len) *out_len = 0;
    if (int32_t rc = ensure_unary(input_len, meta)) return rc;
    if (dim >= (size_t)meta->ndim) return err_invalid_dim(dim, (uint64_t)meta->ndim);
    const uint64_t reduce = meta->shape[dim];
    uint64_t outer, inner, total, out_numel;
    if (int32_t rc = dim_loop_sizes(meta, dim, "argmax overflow", &outer, &inner, &total)) return rc;
    if (!checked_mul(outer, inner, &out_numel)) return err_overflow("argmax overflow");
    if (out_numel == 0) return FTH_OK;
    if (reduce == 0) {
        set_error(FTH_ERR_EMPTY_REDUCTION_DIM, "argmax over dimension %zu of size zero", dim);
        fth::last_error().a = dim;
        return FTH_ERR_EMPTY_REDUCTION_DIM;
    }
    if (out_len) *out_len = (size_t)out_numel;
    if (out == nullptr && out_cap == 0) return FTH_OK;
    if (int32_t rc = check_out(out, out_cap, (size_t)out_numel)) return rc;
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    T *dx, *dy;
    if (int32_t rc = stage_in(sc, input + meta->storage_offset, (size_t)total, &dx)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)out_numel, &dy)) return rc;
    if (int32_t rc = Dev<T>::argmax(dx, (int64_t)outer, (int64_t)reduce, (int64_t)inner, dy)) return rc;
    return fetch(out, dy, (size_t)out_numel);
}

// cross_entropy_forward / _backward (crates/ft-kernel-cpu/src/lib.rs:6717-6781 / 6649-6712). `target` holds class
// indices (the reference's &[usize]); an index >= classes makes the reference panic on the slice index and is
// reported here as InvalidArgument naming the row.
template <typename T>
int32_t cross_entropy_impl(bool backward, const T *logits, size_t logits_len, const uint64_t *target, size_t target_len, const T *dloss,
                           size_t dloss_len, size_t batch, size_t classes, T *out, size_t out_cap) {
    uint64_t total;
    FTH_ARG(checked_mul(batch, classes, &total), "cross_entropy: batch * classes overflows");
    const size_t n_out = backward ? (size_t)total : batch;
    if (int32_t rc = check_out(out, out_cap, n_out)) return rc;
    FTH_ARG(logits_len >= total && target_len >= batch && (!backward || dloss_len >= batch), "cross_entropy: input slice shorter than its shape");
    if (batch == 0) return FTH_OK;
    for (size_t i = 0; i < batch; ++i)
        FTH_ARG(target[i] < classes, "cross_entropy: target %llu of row %zu is outside [0, %zu)", (unsigned long long)target[i], i, classes);
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    T *dl = nullptr, *dg = nullptr, *dout = nullptr;
    int64_t *dt = nullptr;
    if (int32_t rc = stage_in(sc, logits, (size_t)total, &dl)) return rc;
    if (int32_t rc = stage_in(sc, reinterpret_cast<const int64_t *>(target), batch, &dt)) return rc;
    if (backward)
        if (int32_t rc = stage_in(sc, dloss, batch, &dg)) return rc;
    if (int32_t rc = stage_out(sc, n_out, &dout)) return rc;
    if (int32_t rc = backward ? Dev<T>::ce_bwd(dl, dt, dg, (int64_t)batch, (int64_t)classes, dout, nullptr)
                              : Dev<T>::ce_fwd(dl, dt, (int64_t)batch, (int64_t)classes, dout, nullptr))
        return rc;
    return fetch(out, dout, n_out);
}

// quantize_per_output_channel_i8 / quantize_rows_i8 (crates/ft-kernel-cpu/src/lib.rs:37836-37905): the two functions
// are the same arithmetic on the rows of a matrix.
int32_t quantize_i8_impl(const float *w, size_t w_len, size_t rows, size_t cols, int8_t *q, size_t q_cap, float *scales, size_t scales_cap) {
    uint64_t total;
    FTH_ARG(checked_mul(rows, cols, &total), "quantize_i8: rows * cols overflows");
    FTH_ARG(w_len == total, "quantize_i8: slice length %zu must equal rows * cols = %llu", w_len, (unsigned long long)total);
    if (int32_t rc = check_out(q, q_cap, (size_t)total)) return rc;
    if (int32_t rc = check_out(scales, scales_cap, rows)) return rc;
    if (rows == 0) return FTH_OK;
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    float *dw = nullptr, *ds = nullptr;
    int8_t *dq = nullptr;
    if (int32_t rc = stage_in(sc, w, (size_t)total, &dw)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)total, &dq)) return rc;
    if (int32_t rc = stage_out(sc, rows, &ds)) return rc;
    if (int32_t rc = fth_dev_quantize_rows_i8(dw, (int64_t)rows, (int64_t)cols, dq, ds, nullptr)) return rc;
    if (int32_t rc = fetch(q, dq, (size_t)total)) return rc;
    return fetch(scales, ds, rows);
}

// linear_int8_dynamic_f32 (crates/ft-kernel-cpu/src/lib.rs:37966-38060)
int32_t linear_int8_impl(const float *x, size_t x_len, size_t m, size_t k, const int8_t *w_i8, size_t w_len, const float *w_scales,
                         size_t w_scales_len, size_t n, const float *bias, size_t bias_len, float *out, size_t out_cap) {
    uint64_t xn, wn, on;
    FTH_ARG(checked_mul(m, k, &xn) && checked_mul(n, k, &wn) && checked_mul(m, n, &on), "linear_int8: shape product overflows");
    FTH_ARG(x_len == xn, "x length must equal m*k");
    FTH_ARG(w_len == wn, "w_i8 length must equal n*k");
    FTH_ARG(w_scales_len == n, "w_scales length must equal n");
    FTH_ARG(bias == nullptr || bias_len == n, "bias length must equal n");
    if (int32_t rc = check_out(out, out_cap, (size_t)on)) return rc;
    if (on == 0) return FTH_OK;
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    float *dx = nullptr, *dws = nullptr, *db = nullptr, *dout = nullptr;
    int8_t *dw = nullptr;
    void *ws = nullptr;
    if (int32_t rc = stage_in(sc, x, (size_t)xn, &dx)) return rc;
    if (int32_t rc = stage_in(sc, w_i8, (size_t)wn, &dw)) return rc;
    if (int32_t rc = stage_in(sc, w_scales, n, &dws)) return rc;
    if (bias)
        if (int32_t rc = stage_in(sc, bias, n, &db)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)on, &dout)) return rc;
    const size_t ws_bytes = fth_dev_linear_int8_workspace_bytes((int64_t)m, (int64_t)k);
    if (int32_t rc = sc.get(&ws, ws_bytes)) return rc;
    if (int32_t rc = fth_dev_linear_int8_dynamic_f32(dx, (int64_t)m, (int64_t)k, dw, dws, (int64_t)n, db, dout, ws, ws_bytes, nullptr)) return rc;
    return fetch(out, dout, (size_t)on);
}

// ---- backward entry points on host slices ----
// Several outputs per call, each with its own capacity; every output the call produces must fit.
template <typename T> int32_t fetch_no_sync(T *host, const T *dev, size_t n) {
    if (n) FTH_HIP(hipMemcpyAsync(host, dev, n * sizeof(T), hipMemcpyDeviceToHost, fth::resolve_stream(nullptr)));
    return FTH_OK;
}

// layer_norm_backward (crates/ft-kernel-cpu/src/lib.rs:6189-6322 / 6052-6183), rms_norm_backward (:6574-6646 / 6503-6570)
template <typename T, bool RMS>
int32_t norm_backward_impl(const T *dy, size_t dy_len, const T *x, size_t x_len, const T *w, size_t batch, size_t n, T eps, T *dx,
                           size_t dx_cap, T *dw, size_t dw_cap, T *db, size_t db_cap) {
    uint64_t total;
    FTH_ARG(checked_mul(batch, n, &total), "norm backward: batch * norm_size overflows");
    FTH_ARG(RMS || w != nullptr, "layer_norm backward: weight is required");
    const bool want_w = w != nullptr;
    if (int32_t rc = check_out(dx, dx_cap, (size_t)total)) return rc;
    if (want_w)
        if (int32_t rc = check_out(dw, dw_cap, n)) return rc;
    if (!RMS)
        if (int32_t rc = check_out(db, db_cap, n)) return rc;
    FTH_ARG(dy_len >= total && x_len >= total, "norm backward: input slice shorter than batch * norm_size");
    if (n == 0) return FTH_OK;
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    T *ddy = nullptr, *dxin = nullptr, *dwt = nullptr, *ddx = nullptr, *ddw = nullptr, *ddb = nullptr;
    void *ws = nullptr;
    if (int32_t rc = stage_in(sc, dy, (size_t)total, &ddy)) return rc;
    if (int32_t rc = stage_in(sc, x, (size_t)total, &dxin)) return rc;
    if (w)
        if (int32_t rc = stage_in(sc, w, n, &dwt)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)total, &ddx)) return rc;
    if (want_w)
        if (int32_t rc = stage_out(sc, n, &ddw)) return rc;
    if (!RMS)
        if (int32_t rc = stage_out(sc, n, &ddb)) return rc;
    const size_t wsb = fth_dev_norm_backward_workspace_bytes((int64_t)batch, (int64_t)n, Dev<T>::dtype);
    if (int32_t rc = sc.get(&ws, wsb)) return rc;
    int32_t rc;
    if constexpr (std::is_same<T, float>::value) {
        rc = RMS ? fth_dev_rms_norm_backward_f32(ddy, dxin, dwt, (int64_t)batch, (int64_t)n, eps, ddx, ddw, ws, wsb, nullptr)
                 : fth_dev_layer_norm_backward_f32(ddy, dxin, dwt, (int64_t)batch, (int64_t)n, eps, ddx, ddw, ddb, ws, wsb, nullptr);
    } else {
        rc = RMS ? fth_dev_rms_norm_backward_f64(ddy, dxin, dwt, (int64_t)batch, (int64_t)n, eps, ddx, ddw, ws, wsb, nullptr)
                 : fth_dev_layer_norm_backward_f64(ddy, dxin, dwt, (int64_t)batch, (int64_t)n, eps, ddx, ddw, ddb, ws, wsb, nullptr);
    }
    if (rc) return rc;
    if (want_w)
        if (int32_t r2 = fetch_no_sync(dw, ddw, n)) return r2;
    if (!RMS)
        if (int32_t r2 = fetch_no_sync(db, ddb, n)) return r2;
    return fetch(dx, ddx, (size_t)total);
}

// linear_backward (crates/ft-kernel-cpu/src/lib.rs:17226-17302)
template <typename T>
int32_t linear_backward_impl(const T *dy, size_t dy_len, const T *x, size_t x_len, const T *w, size_t w_len, size_t batch, size_t in_f,
                             size_t out_f, int32_t need_bias, T *dx, size_t dx_cap, T *dw, size_t dw_cap, T *db, size_t db_cap) {
    uint64_t n_dy, n_x, n_w;
    FTH_ARG(checked_mul(batch, out_f, &n_dy) && checked_mul(batch, in_f, &n_x) && checked_mul(out_f, in_f, &n_w),
            "linear backward: extents overflow");
    if (int32_t rc = check_out(dx, dx_cap, (size_t)n_x)) return rc;
    if (int32_t rc = check_out(dw, dw_cap, (size_t)n_w)) return rc;
    if (need_bias)
        if (int32_t rc = check_out(db, db_cap, out_f)) return rc;
    FTH_ARG(dy_len >= n_dy && x_len >= n_x && w_len >= n_w, "linear backward: input slice shorter than its shape");
    if (n_x == 0 && n_w == 0 && (!need_bias || out_f == 0)) return FTH_OK;
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    T *ddy = nullptr, *dxin = nullptr, *dwt = nullptr, *ddx = nullptr, *ddw = nullptr, *ddb = nullptr;
    void *ws = nullptr;
    if (int32_t rc = stage_in(sc, dy, (size_t)n_dy, &ddy)) return rc;
    if (int32_t rc = stage_in(sc, x, (size_t)n_x, &dxin)) return rc;
    if (int32_t rc = stage_in(sc, w, (size_t)n_w, &dwt)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)n_x, &ddx)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)n_w, &ddw)) return rc;
    if (need_bias)
        if (int32_t rc = stage_out(sc, out_f, &ddb)) return rc;
    const size_t wsb = fth_dev_linear_backward_workspace_bytes((int64_t)batch, (int64_t)out_f, Dev<T>::dtype);
    if (int32_t rc = sc.get(&ws, wsb)) return rc;
    // dweight of an empty batch is all zeros (the product over k = 0), which the k == 0 GEMM path writes.
    int32_t rc;
    if constexpr (std::is_same<T, float>::value)
        rc = fth_dev_linear_backward_f32(ddy, dxin, dwt, (int64_t)batch, (int64_t)in_f, (int64_t)out_f, ddx, ddw, ddb, ws, wsb, nullptr);
    else
        rc = fth_dev_linear_backward_f64(ddy, dxin, dwt, (int64_t)batch, (int64_t)in_f, (int64_t)out_f, ddx, ddw, ddb, ws, wsb, nullptr);
    if (rc) return rc;
    if (int32_t r2 = fetch_no_sync(dw, ddw, (size_t)n_w)) return r2;
    if (need_bias)
        if (int32_t r2 = fetch_no_sync(db, ddb, out_f)) return r2;
    return fetch(dx, ddx, (size_t)n_x);
}

// sdpa_backward (crates/ft-kernel-cpu/src/lib.rs:5539-5650 / 5300-5414) and sdpa_backward_masked (:5423-5530, `masked`)
template <typename T>
int32_t sdpa_backward_impl(const T *q, size_t q_len, const T *k, size_t k_len, const T *v, size_t v_len, const T *dout, size_t do_len,
                           size_t num_bh, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, T scale, int32_t causal, T *dq,
                           size_t dq_cap, T *dk, size_t dk_cap, T *dv, size_t dv_cap, bool masked = false, const T *mask = nullptr,
                           size_t mask_len = 0, size_t mask_bh_stride = 0, bool unit_dout = false) {
    uint64_t nq, nk, nv, no, t;
    FTH_ARG(checked_mul(num_bh, seq_q, &t) && checked_mul(t, d_k, &nq) && checked_mul(t, d_v, &no) && checked_mul(num_bh, seq_k, &t) &&
                checked_mul(t, d_k, &nk) && checked_mul(t, d_v, &nv),
            "sdpa backward: extents overflow");
    if (int32_t rc = check_out(dq, dq_cap, (size_t)nq)) return rc;
    if (int32_t rc = check_out(dk, dk_cap, (size_t)nk)) return rc;
    if (int32_t rc = check_out(dv, dv_cap, (size_t)nv)) return rc;
    FTH_ARG(q_len >= nq && k_len >= nk && v_len >= nv && (unit_dout || do_len >= no), "sdpa backward: input slice shorter than its shape");
    uint64_t nm = 0;
    if (masked && num_bh > 0 && seq_q > 0 && seq_k > 0) {
        uint64_t plane, span;
        FTH_ARG(checked_mul(seq_q, seq_k, &plane) && checked_mul(num_bh - 1, mask_bh_stride, &span) && span + plane >= span,
                "sdpa backward: mask extents overflow");
        nm = span + plane;
        FTH_ARG(mask_bh_stride == 0 || mask_bh_stride >= plane, "sdpa backward: mask_bh_stride %zu is neither 0 nor >= seq_q * seq_k",
                mask_bh_stride);
        FTH_ARG(mask != nullptr && mask_len >= nm, "sdpa backward: mask slice shorter than (num_bh - 1) * mask_bh_stride + seq_q * seq_k");
    }
    if (nq == 0 && nk == 0 && nv == 0) return FTH_OK;
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    T *dqi = nullptr, *dki = nullptr, *dvi = nullptr, *ddo = nullptr, *gq = nullptr, *gk = nullptr, *gv = nullptr, *dmask = nullptr;
    void *ws = nullptr;
    if (nm > 0)
        if (int32_t rc = stage_in(sc, mask, (size_t)nm, &dmask)) return rc;
    if (int32_t rc = stage_in(sc, q, (size_t)nq, &dqi)) return rc;
    if (int32_t rc = stage_in(sc, k, (size_t)nk, &dki)) return rc;
    if (int32_t rc = stage_in(sc, v, (size_t)nv, &dvi)) return rc;
    if (!unit_dout)
        if (int32_t rc = stage_in(sc, dout, (size_t)no, &ddo)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)nq, &gq)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)nk, &gk)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)nv, &gv)) return rc;
    const size_t wsb = unit_dout ? fth_dev_sdpa_backward_unit_dout_workspace_bytes((int64_t)num_bh, (int64_t)seq_q, (int64_t)seq_k,
                                                                                   (int64_t)d_v, Dev<T>::dtype)
                                 : fth_dev_sdpa_backward_workspace_bytes((int64_t)num_bh, (int64_t)seq_q, (int64_t)seq_k, Dev<T>::dtype);
    if (int32_t rc = sc.get(&ws, wsb)) return rc;
    int32_t rc;
    if constexpr (std::is_same<T, float>::value) {
        rc = unit_dout ? fth_dev_sdpa_backward_unit_dout_f32(dqi, dki, dvi, (int64_t)num_bh, (int64_t)seq_q, (int64_t)seq_k, (int64_t)d_k,
                                                             (int64_t)d_v, scale, causal, gq, gk, gv, ws, wsb, nullptr)
             : masked ? fth_dev_sdpa_backward_masked_f32(dqi, dki, dvi, ddo, (int64_t)num_bh, (int64_t)seq_q, (int64_t)seq_k, (int64_t)d_k,
                                                       (int64_t)d_v, scale, dmask, (int64_t)mask_bh_stride, gq, gk, gv, ws, wsb, nullptr)
                    : fth_dev_sdpa_backward_f32(dqi, dki, dvi, ddo, (int64_t)num_bh, (int64_t)seq_q, (int64_t)seq_k, (int64_t)d_k,
                                                (int64_t)d_v, scale, causal, gq, gk, gv, ws, wsb, nullptr);
    } else {
        rc = unit_dout ? fth_dev_sdpa_backward_unit_dout_f64(dqi, dki, dvi, (int64_t)num_bh, (int64_t)seq_q, (int64_t)seq_k, (int64_t)d_k,
                                                             (int64_t)d_v, scale, causal, gq, gk, gv, ws, wsb, nullptr)
             : masked ? fth_dev_sdpa_backward_masked_f64(dqi, dki, dvi, ddo, (int64_t)num_bh, (int64_t)seq_q, (int64_t)seq_k, (int64_t)d_k,
                                                       (int64_t)d_v, scale, dmask, (int64_t)mask_bh_stride, gq, gk, gv, ws, wsb, nullptr)
                    : fth_dev_sdpa_backward_f64(dqi, dki, dvi, ddo, (int64_t)num_bh, (int64_t)seq_q, (int64_t)seq_k, (int64_t)d_k,
                                                (int64_t)d_v, scale, causal, gq, gk, gv, ws, wsb, nullptr);
    }
    if (rc) return rc;
    if (int32_t r2 = fetch_no_sync(dk, gk, (size_t)nk)) return r2;
    if (int32_t r2 = fetch_no_sync(dv, gv, (size_t)nv)) return r2;
    return fetch(dq, gq, (size_t)nq);
}

// transpose_2d_into_f32 / _f64 (crates/ft-kernel-cpu/src/lib.rs:42415-42439, 42294-42318) and
// transpose_batched_materialize_f32 / _f64 (:42526-42556, 42490-42519): dst[b][c][r] = src[b][r][c]. The reference
// asserts src.len() == dst.len() == batch * rows * cols in debug builds and indexes past a short slice otherwise.
template <typename T>
int32_t transpose_impl(const T *src, size_t src_len, size_t batch, size_t rows, size_t cols, T *out, size_t out_cap) {
    uint64_t plane, total;
    FTH_ARG(checked_mul(rows, cols, &plane) && checked_mul(plane, batch, &total), "transpose: batch * rows * cols overflows");
    if (int32_t rc = check_out(out, out_cap, (size_t)total)) return rc;
    if (total == 0) return FTH_OK;
    FTH_ARG(src != nullptr && src_len >= total, "transpose: source slice shorter than batch * rows * cols");
    FTH_ARG(total <= (uint64_t)std::numeric_limits<int64_t>::max(), "transpose: tensor too large");
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    T *ds, *dd;
    if (int32_t rc = stage_in(sc, src, (size_t)total, &ds)) return rc;
    if (int32_t rc = stage_out(sc, (size_t)total, &dd)) return rc;
    int32_t rc;
    if constexpr (sizeof(T) == 4) rc = fth_dev_transpose_batched_f32(ds, dd, (int64_t)batch, (int64_t)rows, (int64_t)cols, nullptr);
    else rc = fth_dev_transpose_batched_f64(ds, dd, (int64_t)batch, (int64_t)rows, (int64_t)cols, nullptr);
    if (rc) return rc;
    return fetch(out, dd, (size_t)total);
}

}  // namespace

extern "C" {

int32_t fth_matmul_tensor_contiguous_f32(const float *lhs, size_t lhs_len, const float *rhs, size_t rhs_len,
                                         const fth_meta *lm, const fth_meta *rm, float *out, size_t out_cap, size_t *out_len) {
    return matmul_impl<float>(lhs, lhs_len, rhs, rhs_len, lm, rm, out, out_cap, out_len);
}
int32_t fth_matmul_tensor_contiguous_f64(const double *lhs, size_t lhs_len, const double *rhs, size_t rhs_len,
                                         const fth_meta *lm, const fth_meta *rm, double *out, size_t out_cap, size_t *out_len) {
    return matmul_impl<double>(lhs, lhs_len, rhs, rhs_len, lm, rm, out, out_cap, out_len);
}
int32_t fth_bmm_tensor_contiguous_f32(const float *lhs, size_t lhs_len, const float *rhs, size_t rhs_len,
                                      const fth_meta *lm, const fth_meta *rm, float *out, size_t out_cap, size_t *out_len) {
    return bmm_impl<float>(lhs, lhs_len, rhs, rhs_len, lm, rm, out, out_cap, out_len);
}
int32_t fth_bmm_tensor_contiguous_f64(const double *lhs, size_t lhs_len, const double *rhs, size_t rhs_len,
                                      const fth_meta *lm, const fth_meta *rm, double *out, size_t out_cap, size_t *out_len) {
    return bmm_impl<double>(lhs, lhs_len, rhs, rhs_len, lm, rm, out, out_cap, out_len);
}
int32_t fth_addmm_tensor_contiguous_f32(const float *input, size_t input_len, const float *mat1, size_t mat1_len,
                                        const float *mat2, size_t mat2_len, const fth_meta *im, const fth_meta *m1,
                                        const fth_meta *m2, float beta, float alpha, float *out, size_t out_cap, size_t *out_len) {
    return addmm_impl<float>(input, input_len, mat1, mat1_len, mat2, mat2_len, im, m1, m2, beta, alpha, out, out_cap, out_len);
}
int32_t fth_addmm_tensor_contiguous_f64(const double *input, size_t input_len, const double *mat1, size_t mat1_len,
                                        const double *mat2, size_t mat2_len, const fth_meta *im, const fth_meta *m1,
                                        const fth_meta *m2, double beta, double alpha, double *out, size_t out_cap, size_t *out_len) {
    return addmm_impl<double>(input, input_len, mat1, mat1_len, mat2, mat2_len, im, m1, m2, beta, alpha, out, out_cap, out_len);
}
int32_t fth_linear_tensor_f32(const float *x, size_t x_len, const float *w, size_t w_len, const float *bias, size_t bias_len,
                              size_t batch, size_t in_f, size_t out_f, float *out, size_t out_cap, size_t *out_len) {
    return linear_impl<float>(x, x_len, w, w_len, bias, bias_len, batch, in_f, out_f, out, out_cap, out_len);
}
int32_t fth_linear_tensor_f64(const double *x, size_t x_len, const double *w, size_t w_len, const double *bias, size_t bias_len,
                              size_t batch, size_t in_f, size_t out_f, double *out, size_t out_cap, size_t *out_len) {
    return linear_impl<double>(x, x_len, w, w_len, bias, bias_len, batch, in_f, out_f, out, out_cap, out_len);
}
int32_t fth_matmul_rhs_transposed_contiguous_f32(size_t m, size_t k, size_t n, const float *lhs, size_t lhs_len,
                                                 const float *rhs, size_t rhs_len, float *out, size_t out_cap, size_t *out_len) {
    return matmul_bt_impl<float>(m, k, n, lhs, lhs_len, rhs, rhs_len, out, out_cap, out_len);
}
int32_t fth_matmul_rhs_transposed_contiguous_f64(size_t m, size_t k, size_t n, const double *lhs, size_t lhs_len,
                                                 const double *rhs, size_t rhs_len, double *out, size_t out_cap, size_t *out_len) {
    return matmul_bt_impl<double>(m, k, n, lhs, lhs_len, rhs, rhs_len, out, out_cap, out_len);
}
int32_t fth_softmax_dim_tensor_contiguous_f32(const float *input, size_t input_len, const fth_meta *meta, size_t dim,
                                              float *out, size_t out_cap, size_t *out_len) {
    return softmax_impl<float>(input, input_len, meta, dim, out, out_cap, out_len);
}
int32_t fth_softmax_dim_tensor_contiguous_f64(const double *input, size_t input_len, const fth_meta *meta, size_t dim,
                                              double *out, size_t out_cap, size_t *out_len) {
    return softmax_impl<double>(input, input_len, meta, dim, out, out_cap, out_len);
}
int32_t fth_layer_norm_forward_f32(const float *x, size_t x_len, const float *w, const float *b, size_t batch, size_t n,
                                   float eps, float *out, size_t out_cap) {
    return layer_norm_impl<float>(x, nullptr, x_len, w, b, batch, n, eps, out, out_cap);
}
int32_t fth_layer_norm_forward_f64(const double *x, size_t x_len, const double *w, const double *b, size_t batch, size_t n,
                                   double eps, double *out, size_t out_cap) {
    return layer_norm_impl<double>(x, nullptr, x_len, w, b, batch, n, eps, out, out_cap);
}
int32_t fth_add_layer_norm_forward_f32(const float *a, const float *b2, size_t ab_len, const float *w, const float *b,
                                       size_t batch, size_t n, float eps, float *out, size_t out_cap) {
    FTH_ARG(a != nullptr && b2 != nullptr, "add_layer_norm: NULL operand");
    return layer_norm_impl<float>(a, b2, ab_len, w, b, batch, n, eps, out, out_cap);
}
int32_t fth_rms_norm_forward_f32(const float *x, size_t x_len, const float *w, size_t batch, size_t n, float eps,
                                 float *out, size_t out_cap) {
    return rms_norm_impl<float>(x, x_len, w, batch, n, eps, out, out_cap);
}
int32_t fth_rms_norm_forward_f64(const double *x, size_t x_len, const double *w, size_t batch, size_t n, double eps,
                                 double *out, size_t out_cap) {
    return rms_norm_impl<double>(x, x_len, w, batch, n, eps, out, out_cap);
}
int32_t fth_gelu_tensor_contiguous_f32(const float *input, size_t input_len, const fth_meta *meta, float *out,
                                       size_t out_cap, size_t *out_len) {
    return gelu_impl<float>(input, input_len, meta, out, out_cap, out_len);
}
int32_t fth_gelu_tanh_tensor_contiguous_f32(const float *input, size_t input_len, const fth_meta *meta, float *out, size_t out_cap,
                                            size_t *out_len) {
    return gelu_impl<float>(input, input_len, meta, out, out_cap, out_len, true);
}
int32_t fth_gelu_tanh_tensor_contiguous_f64(const double *input, size_t input_len, const fth_meta *meta, double *out, size_t out_cap,
                                            size_t *out_len) {
    return gelu_impl<double>(input, input_len, meta, out, out_cap, out_len, true);
}
int32_t fth_gelu_tensor_contiguous_f64(const double *input, size_t input_len, const fth_meta *meta, double *out,
                                       size_t out_cap, size_t *out_len) {
    return gelu_impl<double>(input, input_len, meta, out, out_cap, out_len);
}
int32_t fth_add_tensor_contiguous_f32(const float *lhs, size_t lhs_len, const float *rhs, size_t rhs_len,
                                      const fth_meta *lm, const fth_meta *rm, float *out, size_t out_cap, size_t *out_len) {
    return add_impl<float>(lhs, lhs_len, rhs, rhs_len, lm, rm, out, out_cap, out_len);
}
int32_t fth_add_tensor_contiguous_f64(const double *lhs, size_t lhs_len, const double *rhs, size_t rhs_len,
                                      const fth_meta *lm, const fth_meta *rm, double *out, size_t out_cap, size_t *out_len) {
    return add_impl<double>(lhs, lhs_len, rhs, rhs_len, lm, rm, out, out_cap, out_len);
}
int32_t fth_sdpa_forward_f32(const float *q, size_t q_len, const float *k, size_t k_len, const float *v, size_t v_len,
                             size_t num_bh, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, float scale,
                             int32_t causal, float *out, size_t out_cap) {
    return sdpa_impl<float>(q, q_len, k, k_len, v, v_len, num_bh, seq_q, seq_k, d_k, d_v, scale, causal, out, out_cap);
}
int32_t fth_sdpa_forward_f64(const double *q, size_t q_len, const double *k, size_t k_len, const double *v, size_t v_len,
                             size_t num_bh, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, double scale,
                             int32_t causal, double *out, size_t out_cap) {
    return sdpa_impl<double>(q, q_len, k, k_len, v, v_len, num_bh, seq_q, seq_k, d_k, d_v, scale, causal, out, out_cap);
}
int32_t fth_index_select_tensor_contiguous_f32(const float *input, size_t input_len, const fth_meta *meta, size_t dim,
                                               const double *indices, size_t num_indices, float *out, size_t out_cap, size_t *out_len) {
    return index_select_impl<float>(input, input_len, meta, dim, indices, num_indices, out, out_cap, out_len);
}
int32_t fth_index_select_tensor_contiguous_f64(const double *input, size_t input_len, const fth_meta *meta, size_t dim,
                                               const double *indices, size_t num_indices, double *out, size_t out_cap, size_t *out_len) {
    return index_select_impl<double>(input, input_len, meta, dim, indices, num_indices, out, out_cap, out_len);
}
int32_t fth_argmax_dim_tensor_contiguous_f32(const float *input, size_t input_len, const fth_meta *meta, size_t dim,
                                             float *out, size_t out_cap, size_t *out_len) {
    return argmax_impl<float>(input, input_len, meta, dim, out, out_cap, out_len);
}
int32_t fth_argmax_dim_tensor_contiguous_f64(const double *input, size_t input_len, const fth_meta *meta, size_t dim,
                                             double *out, size_t out_cap, size_t *out_len) {
    return argmax_impl<double>(input, input_len, meta, dim, out, out_cap, out_len);
}

int32_t fth_layer_norm_backward_f32(const float *dy, size_t dy_len, const float *x, size_t x_len, const float *weight, size_t batch,
                                    size_t norm_size, float eps, float *dx, size_t dx_cap, float *dweight, size_t dweight_cap,
                                    float *dbias, size_t dbias_cap) {
    return norm_backward_impl<float, false>(dy, dy_len, x, x_len, weight, batch, norm_size, eps, dx, dx_cap, dweight, dweight_cap, dbias, dbias_cap);
}
int32_t fth_layer_norm_backward_f64(const double *dy, size_t dy_len, const double *x, size_t x_len, const double *weight, size_t batch,
                                    size_t norm_size, double eps, double *dx, size_t dx_cap, double *dweight, size_t dweight_cap,
                                    double *dbias, size_t dbias_cap) {
    return norm_backward_impl<double, false>(dy, dy_len, x, x_len, weight, batch, norm_size, eps, dx, dx_cap, dweight, dweight_cap, dbias, dbias_cap);
}
int32_t fth_rms_norm_backward_f32(const float *dy, size_t dy_len, const float *x, size_t x_len, const float *weight, size_t batch,
                                  size_t norm_size, float eps, float *dx, size_t dx_cap, float *dweight, size_t dweight_cap) {
    return norm_backward_impl<float, true>(dy, dy_len, x, x_len, weight, batch, norm_size, eps, dx, dx_cap, dweight, dweight_cap, nullptr, 0);
}
int32_t fth_rms_norm_backward_f64(const double *dy, size_t dy_len, const double *x, size_t x_len, const double *weight, size_t batch,
                                  size_t norm_size, double eps, double *dx, size_t dx_cap, double *dweight, size_t dweight_cap) {
    return norm_backward_impl<double, true>(dy, dy_len, x, x_len, weight, batch, norm_size, eps, dx, dx_cap, dweight, dweight_cap, nullptr, 0);
}
int32_t fth_linear_backward_f32(const float *dy, size_t dy_len, const float *x, size_t x_len, const float *weight, size_t weight_len,
                                size_t batch, size_t in_features, size_t out_features, int32_t need_bias, float *dx, size_t dx_cap,
                                float *dweight, size_t dweight_cap, float *dbias, size_t dbias_cap) {
    return linear_backward_impl<float>(dy, dy_len, x, x_len, weight, weight_len, batch, in_features, out_features, need_bias, dx, dx_cap,
                                       dweight, dweight_cap, dbias, dbias_cap);
}
int32_t fth_linear_backward_f64(const double *dy, size_t dy_len, const double *x, size_t x_len, const double *weight, size_t weight_len,
                                size_t batch, size_t in_features, size_t out_features, int32_t need_bias, double *dx, size_t dx_cap,
                                double *dweight, size_t dweight_cap, double *dbias, size_t dbias_cap) {
    return linear_backward_impl<double>(dy, dy_len, x, x_len, weight, weight_len, batch, in_features, out_features, need_bias, dx, dx_cap,
                                        dweight, dweight_cap, dbias, dbias_cap);
}
int32_t fth_sdpa_backward_f32(const float *q, size_t q_len, const float *k, size_t k_len, const float *v, size_t v_len, const float *dout,
                              size_t dout_len, size_t num_bh, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, float scale,
                              int32_t causal, float *dq, size_t dq_cap, float *dk, size_t dk_cap, float *dv, size_t dv_cap) {
    return sdpa_backward_impl<float>(q, q_len, k, k_len, v, v_len, dout, dout_len, num_bh, seq_q, seq_k, d_k, d_v, scale, causal, dq, dq_cap,
                                     dk, dk_cap, dv, dv_cap);
}
int32_t fth_sdpa_backward_f64(const double *q, size_t q_len, const double *k, size_t k_len, const double *v, size_t v_len, const double *dout,
                              size_t dout_len, size_t num_bh, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, double scale,
                              int32_t causal, double *dq, size_t dq_cap, double *dk, size_t dk_cap, double *dv, size_t dv_cap) {
    return sdpa_backward_impl<double>(q, q_len, k, k_len, v, v_len, dout, dout_len, num_bh, seq_q, seq_k, d_k, d_v, scale, causal, dq, dq_cap,
                                      dk, dk_cap, dv, dv_cap);
}
int32_t fth_sdpa_backward_f32_unit_dout(const float *q, size_t q_len, const float *k, size_t k_len, const float *v, size_t v_len, size_t num_bh,
                                        size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, float scale, int32_t causal, float *dq,
                                        size_t dq_cap, float *dk, size_t dk_cap, float *dv, size_t dv_cap) {
    return sdpa_backward_impl<float>(q, q_len, k, k_len, v, v_len, nullptr, 0, num_bh, seq_q, seq_k, d_k, d_v, scale, causal, dq, dq_cap, dk,
                                     dk_cap, dv, dv_cap, false, nullptr, 0, 0, true);
}
int32_t fth_sdpa_backward_masked_f32(const float *q, size_t q_len, const float *k, size_t k_len, const float *v, size_t v_len, const float *dout,
                                     size_t dout_len, size_t num_bh, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, float scale,
                                     const float *mask, size_t mask_len, size_t mask_bh_stride, float *dq, size_t dq_cap, float *dk,
                                     size_t dk_cap, float *dv, size_t dv_cap) {
    return sdpa_backward_impl<float>(q, q_len, k, k_len, v, v_len, dout, dout_len, num_bh, seq_q, seq_k, d_k, d_v, scale, 0, dq, dq_cap, dk,
                                     dk_cap, dv, dv_cap, true, mask, mask_len, mask_bh_stride);
}
int32_t fth_sdpa_backward_masked_f64(const double *q, size_t q_len, const double *k, size_t k_len, const double *v, size_t v_len, const double *dout,
                                     size_t dout_len, size_t num_bh, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, double scale,
                                     const double *mask, size_t mask_len, size_t mask_bh_stride, double *dq, size_t dq_cap, double *dk,
                                     size_t dk_cap, double *dv, size_t dv_cap) {
    return sdpa_backward_impl<double>(q, q_len, k, k_len, v, v_len, dout, dout_len, num_bh, seq_q, seq_k, d_k, d_v, scale, 0, dq, dq_cap, dk,
                                      dk_cap, dv, dv_cap, true, mask, mask_len, mask_bh_stride);
}

int32_t fth_log_softmax_dim_tensor_contiguous_f32(const float *input, size_t input_len, const fth_meta *meta, size_t dim, float *out,
                                                  size_t out_cap, size_t *out_len) {
    return softmax_impl<float>(input, input_len, meta, dim, out, out_cap, out_len, true);
}
int32_t fth_log_softmax_dim_tensor_contiguous_f64(const double *input, size_t input_len, const fth_meta *meta, size_t dim, double *out,
                                                  size_t out_cap, size_t *out_len) {
    return softmax_impl<double>(input, input_len, meta, dim, out, out_cap, out_len, true);
}
int32_t fth_cross_entropy_forward_f32(const float *logits, size_t logits_len, const uint64_t *target, size_t target_len, size_t batch,
                                      size_t classes, float *loss, size_t loss_cap) {
    return cross_entropy_impl<float>(false, logits, logits_len, target, target_len, nullptr, 0, batch, classes, loss, loss_cap);
}
int32_t fth_cross_entropy_forward_f64(const double *logits, size_t logits_len, const uint64_t *target, size_t target_len, size_t batch,
                                      size_t classes, double *loss, size_t loss_cap) {
    return cross_entropy_impl<double>(false, logits, logits_len, target, target_len, nullptr, 0, batch, classes, loss, loss_cap);
}
int32_t fth_cross_entropy_backward_f32(const float *logits, size_t logits_len, const uint64_t *target, size_t target_len, const float *dloss,
                                       size_t dloss_len, size_t batch, size_t classes, float *dlogits, size_t dlogits_cap) {
    return cross_entropy_impl<float>(true, logits, logits_len, target, target_len, dloss, dloss_len, batch, classes, dlogits, dlogits_cap);
}
int32_t fth_cross_entropy_backward_f64(const double *logits, size_t logits_len, const uint64_t *target, size_t target_len, const double *dloss,
                                       size_t dloss_len, size_t batch, size_t classes, double *dlogits, size_t dlogits_cap) {
    return cross_entropy_impl<double>(true, logits, logits_len, target, target_len, dloss, dloss_len, batch, classes, dlogits, dlogits_cap);
}

int32_t fth_sdpa_forward_masked_f32(const float *q, size_t q_len, const float *k, size_t k_len, const float *v, size_t v_len, size_t num_bh,
                                    size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, float scale, const float *mask, size_t mask_len,
                                    size_t mask_bh_stride, float *out, size_t out_cap) {
    return sdpa_masked_impl<float>(q, q_len, k, k_len, v, v_len, num_bh, 1, 1, seq_q, seq_k, d_k, d_v, scale, mask, mask_len, mask_bh_stride, out, out_cap);
}
int32_t fth_sdpa_forward_masked_f64(const double *q, size_t q_len, const double *k, size_t k_len, const double *v, size_t v_len, size_t num_bh,
                                    size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, double scale, const double *mask, size_t mask_len,
                                    size_t mask_bh_stride, double *out, size_t out_cap) {
    return sdpa_masked_impl<double>(q, q_len, k, k_len, v, v_len, num_bh, 1, 1, seq_q, seq_k, d_k, d_v, scale, mask, mask_len, mask_bh_stride, out, out_cap);
}
int32_t fth_sdpa_forward_masked_gqa_f32(const float *q, size_t q_len, const float *k, size_t k_len, const float *v, size_t v_len, size_t batch,
                                        size_t h_q, size_t h_kv, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, float scale,
                                        const float *mask, size_t mask_len, size_t mask_bh_stride, float *out, size_t out_cap) {
    return sdpa_masked_impl<float>(q, q_len, k, k_len, v, v_len, batch, h_q, h_kv, seq_q, seq_k, d_k, d_v, scale, mask, mask_len, mask_bh_stride, out, out_cap);
}
int32_t fth_sdpa_forward_masked_gqa_f64(const double *q, size_t q_len, const double *k, size_t k_len, const double *v, size_t v_len, size_t batch,
                                        size_t h_q, size_t h_kv, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, double scale,
                                        const double *mask, size_t mask_len, size_t mask_bh_stride, double *out, size_t out_cap) {
    return sdpa_masked_impl<double>(q, q_len, k, k_len, v, v_len, batch, h_q, h_kv, seq_q, seq_k, d_k, d_v, scale, mask, mask_len, mask_bh_stride, out, out_cap);
}

int32_t fth_quantize_per_output_channel_i8(const float *w, size_t w_len, size_t rows, size_t cols, int8_t *q, size_t q_cap, float *scales,
                                           size_t scales_cap) {
    return quantize_i8_impl(w, w_len, rows, cols, q, q_cap, scales, scales_cap);
}
int32_t fth_quantize_rows_i8(const float *x, size_t x_len, size_t rows, size_t cols, int8_t *q, size_t q_cap, float *scales, size_t scales_cap) {
    return quantize_i8_impl(x, x_len, rows, cols, q, q_cap, scales, scales_cap);
}
int32_t fth_linear_int8_dynamic_f32(const float *x, size_t x_len, size_t m, size_t k, const int8_t *w_i8, size_t w_len, const float *w_scales,
                                    size_t w_scales_len, size_t n, const float *bias, size_t bias_len, float *out, size_t out_cap) {
    return linear_int8_impl(x, x_len, m, k, w_i8, w_len, w_scales, w_scales_len, n, bias, bias_len, out, out_cap);
}

int32_t fth_transpose_2d_into_f32(const float *src, size_t src_len, float *dst, size_t dst_cap, size_t rows, size_t cols) {
    return transpose_impl<float>(src, src_len, 1, rows, cols, dst, dst_cap);
}
int32_t fth_transpose_2d_into_f64(const double *src, size_t src_len, double *dst, size_t dst_cap, size_t rows, size_t cols) {
    return transpose_impl<double>(src, src_len, 1, rows, cols, dst, dst_cap);
}
int32_t fth_transpose_batched_materialize_f32(const float *src, size_t src_len, size_t batch, size_t rows, size_t cols, float *out,
                                              size_t out_cap) {
    return transpose_impl<float>(src, src_len, batch, rows, cols, out, out_cap);
}
int32_t fth_transpose_batched_materialize_f64(const double *src, size_t src_len, size_t batch, size_t rows, size_t cols, double *out,
                                              size_t out_cap) {
    return transpose_impl<double>(src, src_len, batch, rows, cols, out, out_cap);
}

}  // extern "C"
