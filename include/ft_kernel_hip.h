/*
 * ft_kernel_hip.h -- C ABI of the MI355X (gfx950) kernel backend for the FrankenTorch
 * transformer forward op set.
 *
 * Three tiers, all `extern "C"`, plain pointers and sizes only:
 *
 *   Tier D  (fth_dev_*)   device pointers in, device pointers out, launched on a caller stream.
 *                         This is what a resident runtime (and the benchmark) calls.
 *   Tier A  (fth_*_tensor_contiguous_* / fth_*_forward_* / fth_linear_tensor_*)
 *                         host slices in, caller-provided host buffer out: the shape of the
 *                         `ft_kernel_cpu::*` free functions that `ft-dispatch` routes to
 *                         (crates/ft-dispatch/src/lib.rs:14-250). Each call validates exactly as
 *                         the reference does, uploads, launches Tier D, downloads, synchronises.
 *   Tier B  (fth_tensor_*, fth_batch_*, fth_encoder_*, fth_gpt2_*)
 *                         resident tensors and a stream-ordered batch, the shape of
 *                         `ft_kernel_metal::fused::{GpuTensor, Batch, EncoderGpu}`
 *                         (crates/ft-kernel-metal/src/fused.rs:540-933, 986-1190).
 *
 * Every function returns an `int32_t` status (FTH_OK == 0). Nothing aborts; nothing falls back to
 * a CPU implementation: without a usable HIP device every compute entry point returns
 * FTH_ERR_UNAVAILABLE (the contract of ft_kernel_metal::Error::Unavailable,
 * crates/ft-kernel-metal/src/lib.rs:60-77, 255-272).
 *
 * All tensors are row-major contiguous. Reductions use fixed-order trees (no atomics), so two
 * calls with the same arguments return bitwise identical results.
 */
#ifndef FT_KERNEL_HIP_H
#define FT_KERNEL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------------------------ */
/* Status codes                                                                               */
/* ------------------------------------------------------------------------------------------ */

/* 1..9 mirror `KernelError` (crates/ft-kernel-cpu/src/lib.rs:1697-1733) variant for variant;
 * 100.. mirror `ft_kernel_metal::Error` (crates/ft-kernel-metal/src/lib.rs:60-77);
 * FTH_ERR_INVALID_ARGUMENT stands where the reference's infallible fused entry points would
 * panic on a short slice (plain indexing, e.g. crates/ft-kernel-cpu/src/lib.rs:5888). */
enum {
    FTH_OK = 0,
    FTH_ERR_DTYPE_MISMATCH = 1,        /* Incompatible(DTypeMismatch)   */
    FTH_ERR_DEVICE_MISMATCH = 2,       /* Incompatible(DeviceMismatch)  */
    FTH_ERR_SHAPE_MISMATCH = 3,        /* ShapeMismatch{lhs,rhs}        */
    FTH_ERR_UNSUPPORTED_LAYOUT = 4,    /* UnsupportedLayout{side}       */
    FTH_ERR_STORAGE_SPAN_OVERFLOW = 5, /* StorageSpanOverflow{...}      */
    FTH_ERR_INSUFFICIENT_STORAGE = 6,  /* InsufficientStorage{...}      */
    FTH_ERR_INVALID_DIMENSION = 7,     /* InvalidDimension{dim,ndim}    */
    FTH_ERR_SHAPE_OVERFLOW = 8,        /* ShapeOverflow{context}        */
    FTH_ERR_EMPTY_REDUCTION_DIM = 9,   /* EmptyReductionDim{dim}        */
    FTH_ERR_UNAVAILABLE = 100,         /* Error::Unavailable            */
    FTH_ERR_KERNEL = 101,              /* Error::Kernel(String)         */
    FTH_ERR_SIZE_OVERFLOW = 102,       /* Error::SizeOverflow           */
    FTH_ERR_BUFFER_TOO_LARGE = 103,    /* Error::BufferTooLarge         */
    FTH_ERR_STREAM = 104,              /* Error::CommandBuffer(state)   */
    FTH_ERR_INVALID_ARGUMENT = 105,    /* reference would panic         */
    FTH_ERR_OUTPUT_TOO_SMALL = 106,    /* caller's out buffer < result  */
    FTH_ERR_CORRUPT = 107,             /* TensorIOError::Corrupt{reason} (crates/ft-serialize) */
    FTH_ERR_IO = 108,                  /* TensorIOError::Io{path, source}                     */
    FTH_ERR_INVALID_MAGIC = 109,       /* TensorIOError::InvalidMagic                         */
    FTH_ERR_UNSUPPORTED_VERSION = 110  /* TensorIOError::UnsupportedVersion{found, max}: fth_error_info a = found, b = max */
};

/* DType / Device tags: crates/ft-core/src/lib.rs:23-35 and :176-179, plus the HIP device id the
 * backend adds to `Device`. Only F64 and F32 are computed here (crates/ft-dispatch/src/lib.rs:
 * 4123-4308 narrows F16/BF16 above the kernels). */
enum { FTH_DTYPE_F64 = 0, FTH_DTYPE_F32 = 1, FTH_DTYPE_F16 = 2, FTH_DTYPE_BF16 = 3 }; /* the kernels compute in the first two;
                                                                                       the other two are storage types of a weight file */
enum { FTH_DEVICE_CPU = 0, FTH_DEVICE_CUDA = 1, FTH_DEVICE_HIP = 2 };

#define FTH_MAX_DIMS 8

/* Flattened `TensorMeta` (crates/ft-core/src/lib.rs:340-348). Strides are in elements. */
typedef struct fth_meta {
    int32_t ndim;
    int32_t dtype;  /* FTH_DTYPE_*  */
    int32_t device; /* FTH_DEVICE_* */
    int32_t reserved;
    uint64_t shape[FTH_MAX_DIMS];
    uint64_t strides[FTH_MAX_DIMS];
    uint64_t storage_offset;
} fth_meta;

/* Payload of the last failing call on this thread (the fields of the KernelError variant). */
typedef struct fth_error_info {
    int32_t code;
    int32_t lhs_ndim;
    int32_t rhs_ndim;
    int32_t reserved;
    uint64_t lhs_shape[FTH_MAX_DIMS]; /* ShapeMismatch.lhs */
    uint64_t rhs_shape[FTH_MAX_DIMS]; /* ShapeMismatch.rhs */
    uint64_t a; /* dim | needed | storage_offset | lhs dtype/device tag */
    uint64_t b; /* ndim | available | numel | rhs dtype/device tag      */
    char side[16];     /* "lhs", "rhs", "mat1", "mat2", "input" */
    char message[200]; /* Display-style text, or the HIP error string */
} fth_error_info;

/* Copies the calling thread's last error payload. Returns its code. */
int32_t fth_last_error(fth_error_info *out);
/* Static name for a status code ("ShapeMismatch", "Unavailable", ...). Never NULL. */
const char *fth_status_name(int32_t code);

/* ------------------------------------------------------------------------------------------ */
/* Runtime: availability, memory, streams, timing                                             */
/* ------------------------------------------------------------------------------------------ */

/* ft_kernel_metal::fused::is_available (crates/ft-kernel-metal/src/fused.rs:631-633):
 * 1 when a gfx950 device is present and the kernels in this library can run on it. */
int32_t fth_is_available(void);
/* Fills name (e.g. "gfx950:sramecc+:xnack-"), CU count, HBM bytes, clocks in kHz. */
int32_t fth_device_info(char *arch, size_t arch_cap, int32_t *compute_units, uint64_t *hbm_bytes,
                        int32_t *engine_clock_khz, int32_t *memory_clock_khz);

/* hipMalloc-backed buffers with explicit copies (the `ft-core` storage the backend adds).
 * fth_malloc never zero-fills (crates/ft-kernel-cpu/src/lib.rs:2611-2639 `build_uninit`). */
int32_t fth_malloc(void **dptr, size_t bytes);
int32_t fth_free(void *dptr);
int32_t fth_memcpy_h2d(void *dst_dev, const void *src_host, size_t bytes);
int32_t fth_memcpy_d2h(void *dst_host, const void *src_dev, size_t bytes);
int32_t fth_memcpy_d2d(void *dst_dev, const void *src_dev, size_t bytes);
int32_t fth_memset_zero(void *dst_dev, size_t bytes);
/* Free and total device memory in bytes as the driver reports them (hipMemGetInfo). */
int32_t fth_device_memory_info(uint64_t *free_bytes, uint64_t *total_bytes);
/* Device memory the GEMM unit holds for split-tile accumulators and transposed operands: `live_bytes` in the blocks in
 * use (one per stream and purpose, grown geometrically), `retired_bytes` in outgrown blocks that are kept because
 * queued kernels or a captured graph may still address them (less than `live_bytes` while no single request exceeds
 * 4 GiB). Either pointer may be NULL. The reference's CPU kernels keep no such state. */
int32_t fth_device_workspace_info(uint64_t *live_bytes, uint64_t *retired_bytes);

typedef void *fth_stream; /* a hipStream_t; NULL selects the library's own ordered stream */
typedef void *fth_event;  /* a hipEvent_t */

/* Page-locked host memory (hipHostMalloc) for callers that keep hot tensors in it: the host-slice
 * entry points recognise such slices and let the DMA engines read and write them in place, where
 * an ordinary slice has to be copied through the library's pinned chunks first. No counterpart in
 * the reference (its `Vec<f32>` storage is pageable, crates/ft-core/src/lib.rs:915-925). */
int32_t fth_host_malloc(void **hptr, size_t bytes);
int32_t fth_host_free(void *hptr);
/* Asynchronous copy on stream `s`; kind 1 = host to device, 2 = device to host, 3 = device to
 * device. A host side that is not page-locked makes the copy synchronous with the host. */
int32_t fth_memcpy_async(void *dst, const void *src, size_t bytes, int32_t kind, fth_stream s);
int32_t fth_stream_create(fth_stream *s);
int32_t fth_stream_destroy(fth_stream s);
int32_t fth_stream_synchronize(fth_stream s);
int32_t fth_device_synchronize(void);
int32_t fth_event_create(fth_event *e);
int32_t fth_event_destroy(fth_event e);
int32_t fth_event_record(fth_event e, fth_stream s);
int32_t fth_event_synchronize(fth_event e);
int32_t fth_event_elapsed_ms(fth_event start, fth_event stop, float *ms);

/* ------------------------------------------------------------------------------------------ */
/* Tier D: device-pointer kernels                                                             */
/* ------------------------------------------------------------------------------------------ */

/* Last-dim softmax over `rows` rows of `cols` elements.
 * replaces the inner_size==1 branch of softmax_dim_tensor_contiguous_f32
 * (crates/ft-kernel-cpu/src/lib.rs:39219-39242) / _f64 (:18350-18399). */
int32_t fth_dev_softmax_lastdim_f32(const float *x, float *y, int64_t rows, int64_t cols, fth_stream s);
int32_t fth_dev_softmax_lastdim_f64(const double *x, double *y, int64_t rows, int64_t cols, fth_stream s);
/* Softmax over a middle dim of a contiguous [outer, reduce, inner] view
 * (crates/ft-kernel-cpu/src/lib.rs:39244-39293). */
int32_t fth_dev_softmax_strided_f32(const float *x, float *y, int64_t outer, int64_t reduce, int64_t inner, fth_stream s);
int32_t fth_dev_softmax_strided_f64(const double *x, double *y, int64_t outer, int64_t reduce, int64_t inner, fth_stream s);

/* layer_norm_forward_f32 (crates/ft-kernel-cpu/src/lib.rs:5877-5923), _f64 (:5824-5870).
 * weight / bias may be NULL (the reference's Option::None). */
int32_t fth_dev_layer_norm_f32(const float *x, const float *weight, const float *bias, float *y,
                               int64_t batch, int64_t norm_size, float eps, fth_stream s);
int32_t fth_dev_layer_norm_f64(const double *x, const double *weight, const double *bias, double *y,
                               int64_t batch, int64_t norm_size, double eps, fth_stream s);
/* add_layer_norm_forward_f32 (crates/ft-kernel-cpu/src/lib.rs:5932-5984): y = LN(a + b). */
int32_t fth_dev_add_layer_norm_f32(const float *a, const float *b, const float *weight, const float *bias,
                                   float *y, int64_t batch, int64_t norm_size, float eps, fth_stream s);
/* rms_norm_forward_f32 (crates/ft-kernel-cpu/src/lib.rs:6459-6494), _f64 (:6418-6453). */
int32_t fth_dev_rms_norm_f32(const float *x, const float *weight, float *y, int64_t batch,
                             int64_t norm_size, float eps, fth_stream s);
int32_t fth_dev_rms_norm_f64(const double *x, const double *weight, double *y, int64_t batch,
                             int64_t norm_size, double eps, fth_stream s);

/* gelu_tensor_contiguous_f32 (crates/ft-kernel-cpu/src/lib.rs:37123-37127, 36966-36969): erf form. */
int32_t fth_dev_gelu_f32(const float *x, float *y, int64_t n, fth_stream s);
int32_t fth_dev_gelu_f64(const double *x, double *y, int64_t n, fth_stream s);
/* tanh-form GELU 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))): the `gelu` kernel of the reference's fused GPU module
 * (crates/ft-kernel-metal/src/fused.rs:301-313; f32 keeps its |x| >= 10 clamp) and GELU::tanh()
 * (crates/ft-nn/src/lib.rs:1924-1957, golden values :21985-22004). */
int32_t fth_dev_gelu_tanh_f32(const float *x, float *y, int64_t n, fth_stream s);
int32_t fth_dev_gelu_tanh_f64(const double *x, double *y, int64_t n, fth_stream s);
/* add_tensor_contiguous_f32 (crates/ft-kernel-cpu/src/lib.rs:36870-36877): exact IEEE l + r. */
int32_t fth_dev_add_f32(const float *a, const float *b, float *y, int64_t n, fth_stream s);
int32_t fth_dev_add_f64(const double *a, const double *b, double *y, int64_t n, fth_stream s);
/* The materialising copy behind contiguous / narrow / expand (`copy_from_slice` into a `build_uninit` buffer,
 * crates/ft-kernel-cpu/src/lib.rs:2585-2639): y[i] = x[i], one 128-bit vector per lane, streaming both ways. It is also
 * what the benchmark times as the ceiling of a read-once / write-once kernel on this part. */
int32_t fth_dev_copy_f32(const float *x, float *y, int64_t n, fth_stream s);
int32_t fth_dev_copy_f64(const double *x, double *y, int64_t n, fth_stream s);
/* The bias pass of linear_tensor_f32 (crates/ft-kernel-cpu/src/lib.rs:17336-17351):
 * y[r, j] = x[r, j] + bias[j]. x == y is allowed. */
int32_t fth_dev_bias_add_f32(const float *x, const float *bias, float *y, int64_t rows, int64_t cols, fth_stream s);
int32_t fth_dev_bias_add_f64(const double *x, const double *bias, double *y, int64_t rows, int64_t cols, fth_stream s);
/* Bias pass followed by the residual add, in one sweep with the same two roundings:
 * y[r, j] = (x[r, j] + bias[j]) + residual[r, j]
 * (crates/ft-kernel-cpu/src/lib.rs:17336-17351 then :36870-36877). */
int32_t fth_dev_bias_residual_add_f32(const float *x, const float *bias, const float *residual, float *y,
                                      int64_t rows, int64_t cols, fth_stream s);
int32_t fth_dev_bias_residual_add_f64(const double *x, const double *bias, const double *residual, double *y,
                                      int64_t rows, int64_t cols, fth_stream s);

/* index_select along dim 0 of a [table_rows, width] table: the embedding gather of
 * index_select_tensor_contiguous_f32 (crates/ft-kernel-cpu/src/lib.rs:40216-40253). Indices are
 * f64 VALUES on the device, validated by normalize_strict_index_value's rules
 * (crates/ft-kernel-cpu/src/lib.rs:20058-20090). `bad_index` (device, one int64, may be NULL)
 * receives the smallest position of an invalid index, or -1; rows with an invalid index are
 * left untouched. General [outer, dim, inner] form: fth_dev_index_select_f32. */
int32_t fth_dev_index_select_f32(const float *input, int64_t outer, int64_t dim_size, int64_t inner,
                                 const double *indices, int64_t num_indices, float *out,
                                 int64_t *bad_index, fth_stream s);
int32_t fth_dev_index_select_f64(const double *input, int64_t outer, int64_t dim_size, int64_t inner,
                                 const double *indices, int64_t num_indices, double *out,
                                 int64_t *bad_index, fth_stream s);
/* Fused token + position embedding: out[t, :] = wte[ids[t], :] + wpe[t % seq, :]
 * (Embedding::forward crates/ft-nn/src/lib.rs:3080-3135 twice, then add_tensor_contiguous_f32). */
int32_t fth_dev_embedding_add_f32(const float *wte, int64_t vocab, const float *wpe, int64_t max_pos,
                                  const double *ids, int64_t tokens, int64_t seq, int64_t width,
                                  float *out, int64_t *bad_index, fth_stream s);

/* argmax over the reduce dim of a contiguous [outer, reduce, inner] view; indices are written as
 * floating-point values; first strict maximum wins, the first NaN wins and ends the scan
 * (crates/ft-kernel-cpu/src/lib.rs:39443-39550; f64 :18653). */
int32_t fth_dev_argmax_f32(const float *x, int64_t outer, int64_t reduce, int64_t inner, float *out, fth_stream s);
int32_t fth_dev_argmax_f64(const double *x, int64_t outer, int64_t reduce, int64_t inner, double *out, fth_stream s);
/* logits = x . w^T (x [rows, in_features], w [out_features, in_features], both contiguous) and argmax[r] = the argmax of
 * row r of those logits, by the rule above, in one pass over the logits: the linear product of a greedy decoding step
 * (Linear::forward without bias, crates/ft-nn/src/lib.rs:2965-3010, then argmax_dim :39443). With a workspace of
 * fth_dev_linear_argmax_workspace_floats(rows, out_features) floats (device memory, contents ignored and overwritten) the
 * product's epilogue records the maximum of each row over every 64-column group and the argmax kernel reads those and a
 * few 64-column pieces of the logits instead of every row again; with workspace NULL or smaller, or for shapes the
 * large-tile product kernel does not take, fth_dev_gemm_f32 and fth_dev_argmax_f32 run one after the other. The indices
 * are the same either way, bit for bit those fth_dev_argmax_f32 gives on the logits written here. */
int64_t fth_dev_linear_argmax_workspace_floats(int64_t rows, int64_t out_features);
int32_t fth_dev_linear_argmax_f32(const float *x, const float *w, int64_t rows, int64_t out_features, int64_t in_features,
                                  float *logits, float *argmax, float *workspace, int64_t workspace_floats, fth_stream s);

/* Head split / merge: dst[((b*H+h)*S+s)*hd+c] = src[((b*S+s)*H+h)*hd+c] and its inverse
 * (TensorTape::permute_slice, perm [0,2,1,3], crates/ft-autograd/src/lib.rs:10733-10882). */
int32_t fth_dev_permute_0213_f32(const float *src, float *dst, int64_t d0, int64_t d1, int64_t d2, int64_t d3, fth_stream s);
int32_t fth_dev_permute_0213_f64(const double *src, double *dst, int64_t d0, int64_t d1, int64_t d2, int64_t d3, fth_stream s);

/* 2-D and batched 2-D transposes: dst[b][c][r] = src[b][r][c] for `batch` row-major [rows, cols] planes
 * (transpose_2d_into_f32 / _f64, crates/ft-kernel-cpu/src/lib.rs:42415-42439, 42294-42318;
 * transpose_batched_materialize_f32 / _f64, :42526-42556, 42490-42519). Exact copies of the bits; dst must not be src. */
int32_t fth_dev_transpose_2d_f32(const float *src, float *dst, int64_t rows, int64_t cols, fth_stream s);
int32_t fth_dev_transpose_2d_f64(const double *src, double *dst, int64_t rows, int64_t cols, fth_stream s);
int32_t fth_dev_transpose_batched_f32(const float *src, float *dst, int64_t batch, int64_t rows, int64_t cols, fth_stream s);
int32_t fth_dev_transpose_batched_f64(const double *src, double *dst, int64_t batch, int64_t rows, int64_t cols, fth_stream s);

/* Dense contraction on MFMA. C[b] = alpha * A[b] * op(B[b]) (+ epilogue), beta = 0 (C is fully
 * overwritten, crates/ft-kernel-cpu/src/lib.rs:1310-1338).
 *   trans_b == 0: B is [k, n] row-major         -> gemm::sgemm / dgemm   (:1310, :107)
 *   trans_b == 1: B is [n, k] row-major (W)     -> gemm::sgemm_bt / dgemm_bt (:1430, :201)
 * lda/ldb/ldc are row pitches in elements; batch strides in elements (0 = shared operand).
 * Epilogue, applied to the rounded product in this order (each its own rounding):
 *   FTH_EPI_BIAS      + bias[n]             (linear_tensor_f32, :17336-17351)
 *   FTH_EPI_GELU      gelu_erf(.)           (:36966-36969)
 *   FTH_EPI_GELU_TANH gelu_tanh(.) in place of gelu_erf (crates/ft-kernel-metal/src/fused.rs:301-313; not with FTH_EPI_GELU)
 *   FTH_EPI_RESIDUAL  + residual[m, n]      (row pitch ldc; add_tensor_contiguous_f32)
 * k == 0 writes zeros (or the epilogue of zero); m == 0 or n == 0 returns at once. */
enum { FTH_EPI_NONE = 0, FTH_EPI_BIAS = 1, FTH_EPI_GELU = 2, FTH_EPI_RESIDUAL = 4, FTH_EPI_GELU_TANH = 8 };
typedef struct fth_gemm_desc {
    int64_t m, n, k;
    int64_t lda, ldb, ldc;
    int64_t batch;
    int64_t stride_a, stride_b, stride_c;
    int32_t trans_b;
    int32_t epilogue; /* bit set of FTH_EPI_* */
    int32_t trans_a;  /* 1: A is [k, m] row-major (lda >= m) -> gemm::sgemm_tb / dgemm_tb (:1484, :262); not with trans_b */
    int32_t reserved; /* 0 */
} fth_gemm_desc;
int32_t fth_dev_gemm_f32(const fth_gemm_desc *d, float alpha, const float *a, const float *b, float *c,
                         const float *bias, const float *residual, fth_stream s);
int32_t fth_dev_gemm_f64(const fth_gemm_desc *d, double alpha, const double *a, const double *b, double *c,
                         const double *bias, const double *residual, fth_stream s);

/* log-softmax over the middle dim of a contiguous [outer, reduce, inner] view (inner == 1: the last dim)
 * (log_softmax_dim_tensor_contiguous_f32 / _f64, crates/ft-kernel-cpu/src/lib.rs:39298-39375, 18504-18590). */
int32_t fth_dev_log_softmax_strided_f32(const float *x, float *y, int64_t outer, int64_t reduce, int64_t inner, fth_stream s);
int32_t fth_dev_log_softmax_strided_f64(const double *x, double *y, int64_t outer, int64_t reduce, int64_t inner, fth_stream s);
/* Fused softmax-cross-entropy over [batch, classes] logits with int64 class indices
 * (cross_entropy_forward_f32 / _f64 :6717-6738, 6649-6671; cross_entropy_backward_f32 / _f64 :6745-6781, 6679-6712):
 * loss[i] = lse(logits[i]) - logits[i][target[i]]; dlogits[i][c] = dloss[i] * (softmax(logits[i])[c] - [c == target[i]]).
 * bad_index (may be NULL) receives the lowest row whose target is outside [0, classes), or -1; such rows are not written. */
int32_t fth_dev_cross_entropy_forward_f32(const float *logits, const int64_t *target, int64_t batch, int64_t classes, float *loss,
                                          int64_t *bad_index, fth_stream s);
int32_t fth_dev_cross_entropy_forward_f64(const double *logits, const int64_t *target, int64_t batch, int64_t classes, double *loss,
                                          int64_t *bad_index, fth_stream s);
int32_t fth_dev_cross_entropy_backward_f32(const float *logits, const int64_t *target, const float *dloss, int64_t batch, int64_t classes,
                                           float *dlogits, int64_t *bad_index, fth_stream s);
int32_t fth_dev_cross_entropy_backward_f64(const double *logits, const int64_t *target, const double *dloss, int64_t batch, int64_t classes,
                                           double *dlogits, int64_t *bad_index, fth_stream s);

/* Int8 dynamic-quantised linear (quantize_rows_i8, crates/ft-kernel-cpu/src/lib.rs:37879-37905; quantize_per_output_channel_i8
 * :37836-37868, the same arithmetic on weight rows; linear_int8_dynamic_f32 :37966-38060). Quantisation is per row, symmetric:
 * scale = max|row| / 127 (1 for an all-zero row), q = clamp(round_ties_even(v / scale), -127, 127). The product accumulates
 * in int32 on the integer matrix cores and each output is (float)acc * a_scale[row] * w_scale[col] (+ bias[col]): bit-exact
 * against the reference for any summation order. `fth_dev_linear_int8_dynamic_f32` quantises x into the workspace
 * (fth_dev_linear_int8_workspace_bytes(m, k) bytes) and multiplies; `_prequantized_` takes activations quantised earlier. */
int32_t fth_dev_quantize_rows_i8(const float *x, int64_t rows, int64_t cols, int8_t *q, float *scales, fth_stream s);
size_t fth_dev_linear_int8_workspace_bytes(int64_t m, int64_t k);
int32_t fth_dev_linear_int8_dynamic_f32(const float *x, int64_t m, int64_t k, const int8_t *w_i8, const float *w_scales, int64_t n,
                                        const float *bias, float *out, void *workspace, size_t workspace_bytes, fth_stream s);
int32_t fth_dev_linear_int8_prequantized_f32(const int8_t *x_i8, const float *a_scales, int64_t m, int64_t k, const int8_t *w_i8,
                                             const float *w_scales, int64_t n, const float *bias, float *out, fth_stream s);

/* ---- backward kernels of the same ops (device pointers; caller-provided workspace) ----
 * Each entry point needs scratch memory for its fixed-order partial sums (and, for SDPA, for the
 * probability and score-gradient matrices the reference materialises per head): ask the matching
 * *_workspace_bytes function and pass a device buffer of at least that size. dtype is FTH_DTYPE_*. */

/* layer_norm_backward_f32 / _f64 (crates/ft-kernel-cpu/src/lib.rs:6189-6322, 6052-6183): dy, x, dx are
 * [rows, cols]; weight, dweight, dbias are [cols]; mean / rstd are recomputed from x. */
size_t fth_dev_norm_backward_workspace_bytes(int64_t rows, int64_t cols, int32_t dtype);
int32_t fth_dev_layer_norm_backward_f32(const float *dy, const float *x, const float *weight, int64_t rows, int64_t cols, float eps,
                                        float *dx, float *dweight, float *dbias, void *workspace, size_t workspace_bytes,
                                        fth_stream s);
int32_t fth_dev_layer_norm_backward_f64(const double *dy, const double *x, const double *weight, int64_t rows, int64_t cols, double eps,
                                        double *dx, double *dweight, double *dbias, void *workspace, size_t workspace_bytes,
                                        fth_stream s);
/* LayerNorm backward that allocates nothing. No counterpart in the reference: it is for callers
 * that cannot call hipMalloc (code under HIP graph capture, tight serving loops, harnesses that
 * forbid it) and do not want to carry a workspace. Same kernels and results as
 * fth_dev_layer_norm_backward_f32, with the partial column sums in a device array built into the
 * library (fth_dev_layer_norm_backward_noalloc_max_bytes() = 24 MiB per GPU, held until the process
 * ends). Shapes whose fth_dev_norm_backward_workspace_bytes exceeds that return
 * FTH_ERR_BUFFER_TOO_LARGE (fp32 [8192, 4096] needs 8.1 MiB, [16384, 8192] 16.1 MiB; ask
 * fth_dev_norm_backward_workspace_bytes). All calls on one GPU share the array: calls that overlap
 * in time on one GPU, on any streams, race. The first call on a device looks the array's address
 * up (hipGetSymbolAddress), so make it outside any stream capture; later calls only launch kernels. */
size_t fth_dev_layer_norm_backward_noalloc_max_bytes(void);
int32_t fth_dev_layer_norm_backward_f32_noalloc(const float *dy, const float *x, const float *weight, int64_t rows, int64_t cols, float eps,
                                                float *dx, float *dweight, float *dbias, fth_stream s);
/* rms_norm_backward_f32 / _f64 (:6574-6646, 6503-6570): weight and dweight may both be NULL. */
int32_t fth_dev_rms_norm_backward_f32(const float *dy, const float *x, const float *weight, int64_t rows, int64_t cols, float eps,
                                      float *dx, float *dweight, void *workspace, size_t workspace_bytes, fth_stream s);
int32_t fth_dev_rms_norm_backward_f64(const double *dy, const double *x, const double *weight, int64_t rows, int64_t cols, double eps,
                                      double *dx, double *dweight, void *workspace, size_t workspace_bytes, fth_stream s);

/* linear_backward_f64 (:17226-17302) and the same formulas in f32: dy [batch, out], x [batch, in],
 * weight [out, in] -> dx = dy . weight [batch, in], dweight = dy^T . x [out, in],
 * dbias = column sums of dy [out] (skipped when dbias is NULL, the reference's need_bias = false). */
size_t fth_dev_linear_backward_workspace_bytes(int64_t batch, int64_t out_features, int32_t dtype);
int32_t fth_dev_linear_backward_f32(const float *dy, const float *x, const float *weight, int64_t batch, int64_t in_features,
                                    int64_t out_features, float *dx, float *dweight, float *dbias, void *workspace,
                                    size_t workspace_bytes, fth_stream s);
int32_t fth_dev_linear_backward_f64(const double *dy, const double *x, const double *weight, int64_t batch, int64_t in_features,
                                    int64_t out_features, double *dx, double *dweight, double *dbias, void *workspace,
                                    size_t workspace_bytes, fth_stream s);

/* sdpa_backward_f32 / _f64 (:5539-5650, 5300-5414): contiguous q [num_bh, seq_q, d_k], k [num_bh, seq_k, d_k],
 * v [num_bh, seq_k, d_v], dout [num_bh, seq_q, d_v] -> dq, dk, dv of the shapes of q, k, v. */
size_t fth_dev_sdpa_backward_workspace_bytes(int64_t num_bh, int64_t seq_q, int64_t seq_k, int32_t dtype);
int32_t fth_dev_sdpa_backward_f32(const float *q, const float *k, const float *v, const float *dout, int64_t num_bh, int64_t seq_q,
                                  int64_t seq_k, int64_t d_k, int64_t d_v, float scale, int32_t causal, float *dq, float *dk,
                                  float *dv, void *workspace, size_t workspace_bytes, fth_stream s);
int32_t fth_dev_sdpa_backward_f64(const double *q, const double *k, const double *v, const double *dout, int64_t num_bh, int64_t seq_q,
                                  int64_t seq_k, int64_t d_k, int64_t d_v, double scale, int32_t causal, double *dq, double *dk,
                                  double *dv, void *workspace, size_t workspace_bytes, fth_stream s);
/* sdpa_backward_f32_unit_dout (:5662-5770) and an f64 twin: the backward for dOut = ones([num_bh, seq_q, d_v]) without that
 * tensor (one shared [seq_q, d_v] plane of ones lives in the workspace, which is this much larger than the general form's). */
size_t fth_dev_sdpa_backward_unit_dout_workspace_bytes(int64_t num_bh, int64_t seq_q, int64_t seq_k, int64_t d_v, int32_t dtype);
int32_t fth_dev_sdpa_backward_unit_dout_f32(const float *q, const float *k, const float *v, int64_t num_bh, int64_t seq_q, int64_t seq_k,
                                            int64_t d_k, int64_t d_v, float scale, int32_t causal, float *dq, float *dk, float *dv,
                                            void *workspace, size_t workspace_bytes, fth_stream s);
int32_t fth_dev_sdpa_backward_unit_dout_f64(const double *q, const double *k, const double *v, int64_t num_bh, int64_t seq_q, int64_t seq_k,
                                            int64_t d_k, int64_t d_v, double scale, int32_t causal, double *dq, double *dk, double *dv,
                                            void *workspace, size_t workspace_bytes, fth_stream s);
/* sdpa_backward_masked_f64 (:5423-5530; the same formulas in f32): the recomputed P is softmax(scale * Q.K^T + mask) per row,
 * mask [seq_q, seq_k] rows shared by every (batch, head) when mask_bh_stride == 0, else mask_bh_stride elements apart
 * (>= seq_q * seq_k); the mask is a constant (no gradient). Same workspace as the unmasked form. */
int32_t fth_dev_sdpa_backward_masked_f32(const float *q, const float *k, const float *v, const float *dout, int64_t num_bh, int64_t seq_q,
                                         int64_t seq_k, int64_t d_k, int64_t d_v, float scale, const float *mask, int64_t mask_bh_stride,
                                         float *dq, float *dk, float *dv, void *workspace, size_t workspace_bytes, fth_stream s);
int32_t fth_dev_sdpa_backward_masked_f64(const double *q, const double *k, const double *v, const double *dout, int64_t num_bh, int64_t seq_q,
                                         int64_t seq_k, int64_t d_k, int64_t d_v, double scale, const double *mask, int64_t mask_bh_stride,
                                         double *dq, double *dk, double *dv, void *workspace, size_t workspace_bytes, fth_stream s);

/* Fused scaled-dot-product attention forward, q [num_bh, seq_q, d_k], k [num_bh, seq_k, d_k],
 * v [num_bh, seq_k, d_v] -> out [num_bh, seq_q, d_v]; causal limit = min(qi + 1, seq_k)
 * (sdpa_forward_f32, crates/ft-kernel-cpu/src/lib.rs:5200-5284; _f64 :4572-4651).
 * Row pitches let the kernel read a packed [tokens, 3*d_model] QKV projection and write a
 * [tokens, d_model] context directly (the head split/merge of MultiheadAttention::
 * forward_qkv_masked, crates/ft-nn/src/lib.rs:5088-5198, without the permuted copies):
 * element (bh, s, c) of q lives at q[(bh / heads) * q_batch_stride + (bh % heads) * q_head_stride
 * + s * q_row_stride + c]; likewise k, v, out. */
typedef struct fth_sdpa_desc {
    int64_t num_bh, heads; /* heads divides num_bh; heads == 1 for plain [num_bh, seq, d] */
    int64_t seq_q, seq_k, d_k, d_v;
    int64_t q_batch_stride, q_head_stride, q_row_stride;
    int64_t k_batch_stride, k_head_stride, k_row_stride;
    int64_t v_batch_stride, v_head_stride, v_row_stride;
    int64_t o_batch_stride, o_head_stride, o_row_stride;
    int32_t causal;
    int32_t kv_group; /* grouped-query attention: query heads per K/V head (query head h reads K/V head h / kv_group
                         through k_head_stride / v_head_stride); 0 or 1: one K/V head per query head */
} fth_sdpa_desc;
/* Fills the strides for contiguous [num_bh, seq, d] operands. */
void fth_sdpa_desc_contiguous(fth_sdpa_desc *d, int64_t num_bh, int64_t seq_q, int64_t seq_k,
                              int64_t d_k, int64_t d_v, int32_t causal);
int32_t fth_dev_sdpa_forward_f32(const fth_sdpa_desc *d, float scale, const float *q, const float *k,
                                 const float *v, float *out, fth_stream s);
int32_t fth_dev_sdpa_forward_f64(const fth_sdpa_desc *d, double scale, const double *q, const double *k,
                                 const double *v, double *out, fth_stream s);
/* The same with an additive mask: score * scale + mask[bh * mask_bh_stride + qi * seq_k + key] before the softmax
 * (sdpa_forward_masked_f64, crates/ft-kernel-cpu/src/lib.rs:4661-4741; with kv_group > 1 in the descriptor it is
 * sdpa_forward_masked_gqa_f64, :4777-4850; the reference has the f64 forms only). mask_bh_stride is 0 for one
 * [seq_q, seq_k] mask shared by every (batch, head), else the distance between the masks of consecutive bh
 * (seq_q * seq_k for a packed [num_bh, seq_q, seq_k] mask). -inf hides a key; a row whose every key is hidden is NaN,
 * as in the reference. */
int32_t fth_dev_sdpa_forward_masked_f32(const fth_sdpa_desc *d, float scale, const float *q, const float *k, const float *v,
                                        const float *mask, int64_t mask_bh_stride, float *out, fth_stream s);
int32_t fth_dev_sdpa_forward_masked_f64(const fth_sdpa_desc *d, double scale, const double *q, const double *k, const double *v,
                                        const double *mask, int64_t mask_bh_stride, double *out, fth_stream s);

/* ------------------------------------------------------------------------------------------ */
/* Tier A: host slices in, host buffer out (the ft_kernel_cpu surface)                        */
/* ------------------------------------------------------------------------------------------ */
/* `*_len` are slice lengths in elements. `out` must hold `out_cap` elements; `*out_len` receives
 * the result length (the length of the Vec the reference returns). A NULL `out` with out_cap 0
 * only validates and reports `*out_len`. Validation order follows the reference
 * (crates/ft-kernel-cpu/src/lib.rs:36935-36962, 37787-37793). */

/* matmul_tensor_contiguous_f32 (:37752) / _f64 (:17355) */
int32_t fth_matmul_tensor_contiguous_f32(const float *lhs, size_t lhs_len, const float *rhs, size_t rhs_len,
                                         const fth_meta *lhs_meta, const fth_meta *rhs_meta,
                                         float *out, size_t out_cap, size_t *out_len);
int32_t fth_matmul_tensor_contiguous_f64(const double *lhs, size_t lhs_len, const double *rhs, size_t rhs_len,
                                         const fth_meta *lhs_meta, const fth_meta *rhs_meta,
                                         double *out, size_t out_cap, size_t *out_len);
/* bmm_tensor_contiguous_f32 (:38496) / _f64 (:17785) */
int32_t fth_bmm_tensor_contiguous_f32(const float *lhs, size_t lhs_len, const float *rhs, size_t rhs_len,
                                      const fth_meta *lhs_meta, const fth_meta *rhs_meta,
                                      float *out, size_t out_cap, size_t *out_len);
int32_t fth_bmm_tensor_contiguous_f64(const double *lhs, size_t lhs_len, const double *rhs, size_t rhs_len,
                                      const fth_meta *lhs_meta, const fth_meta *rhs_meta,
                                      double *out, size_t out_cap, size_t *out_len);
/* addmm_tensor_contiguous_f32 (:41562) / _f64 (:17514) */
int32_t fth_addmm_tensor_contiguous_f32(const float *input, size_t input_len, const float *mat1, size_t mat1_len,
                                        const float *mat2, size_t mat2_len, const fth_meta *input_meta,
                                        const fth_meta *mat1_meta, const fth_meta *mat2_meta, float beta,
                                        float alpha, float *out, size_t out_cap, size_t *out_len);
int32_t fth_addmm_tensor_contiguous_f64(const double *input, size_t input_len, const double *mat1, size_t mat1_len,
                                        const double *mat2, size_t mat2_len, const fth_meta *input_meta,
                                        const fth_meta *mat1_meta, const fth_meta *mat2_meta, double beta,
                                        double alpha, double *out, size_t out_cap, size_t *out_len);
/* linear_tensor_f32 (:17306) / _f64 (:17162); bias may be NULL */
int32_t fth_linear_tensor_f32(const float *x, size_t x_len, const float *weight, size_t weight_len,
                              const float *bias, size_t bias_len, size_t batch, size_t in_features,
                              size_t out_features, float *out, size_t out_cap, size_t *out_len);
int32_t fth_linear_tensor_f64(const double *x, size_t x_len, const double *weight, size_t weight_len,
                              const double *bias, size_t bias_len, size_t batch, size_t in_features,
                              size_t out_features, double *out, size_t out_cap, size_t *out_len);
/* matmul_rhs_transposed_contiguous_f32 (:17408) / _f64 (:17381) */
int32_t fth_matmul_rhs_transposed_contiguous_f32(size_t m, size_t k, size_t n, const float *lhs, size_t lhs_len,
                                                 const float *rhs_nk, size_t rhs_len, float *out,
                                                 size_t out_cap, size_t *out_len);
int32_t fth_matmul_rhs_transposed_contiguous_f64(size_t m, size_t k, size_t n, const double *lhs, size_t lhs_len,
                                                 const double *rhs_nk, size_t rhs_len, double *out,
                                                 size_t out_cap, size_t *out_len);
/* softmax_dim_tensor_contiguous_f32 (:39193) / _f64 (:18350) */
int32_t fth_softmax_dim_tensor_contiguous_f32(const float *input, size_t input_len, const fth_meta *meta,
                                              size_t dim, float *out, size_t out_cap, size_t *out_len);
int32_t fth_softmax_dim_tensor_contiguous_f64(const double *input, size_t input_len, const fth_meta *meta,
                                              size_t dim, double *out, size_t out_cap, size_t *out_len);
/* layer_norm_forward_f32 (:5877) / _f64 (:5824); add_layer_norm_forward_f32 (:5932);
 * rms_norm_forward_f32 (:6459) / _f64 (:6418). weight/bias may be NULL. */
int32_t fth_layer_norm_forward_f32(const float *x, size_t x_len, const float *weight, const float *bias,
                                   size_t batch, size_t norm_size, float eps, float *out, size_t out_cap);
int32_t fth_layer_norm_forward_f64(const double *x, size_t x_len, const double *weight, const double *bias,
                                   size_t batch, size_t norm_size, double eps, double *out, size_t out_cap);
int32_t fth_add_layer_norm_forward_f32(const float *a, const float *b, size_t ab_len, const float *weight,
                                       const float *bias, size_t batch, size_t norm_size, float eps,
                                       float *out, size_t out_cap);
int32_t fth_rms_norm_forward_f32(const float *x, size_t x_len, const float *weight, size_t batch,
                                 size_t norm_size, float eps, float *out, size_t out_cap);
int32_t fth_rms_norm_forward_f64(const double *x, size_t x_len, const double *weight, size_t batch,
                                 size_t norm_size, double eps, double *out, size_t out_cap);
/* quantize_per_output_channel_i8 (:37836) / quantize_rows_i8 (:37879): w [rows, cols] -> q [rows * cols], scales [rows].
 * linear_int8_dynamic_f32 (:37966): x [m, k] f32, w_i8 [n, k], w_scales [n], bias [n] or NULL -> out [m * n]. Slice lengths
 * that the reference asserts (x_len == m*k, ...) are InvalidArgument when they differ. */
int32_t fth_quantize_per_output_channel_i8(const float *w, size_t w_len, size_t rows, size_t cols, int8_t *q, size_t q_cap, float *scales,
                                           size_t scales_cap);
int32_t fth_quantize_rows_i8(const float *x, size_t x_len, size_t rows, size_t cols, int8_t *q, size_t q_cap, float *scales, size_t scales_cap);
int32_t fth_linear_int8_dynamic_f32(const float *x, size_t x_len, size_t m, size_t k, const int8_t *w_i8, size_t w_len, const float *w_scales,
                                    size_t w_scales_len, size_t n, const float *bias, size_t bias_len, float *out, size_t out_cap);
/* sdpa_forward_masked_f64 (:4661-4741) and sdpa_forward_masked_gqa_f64 (:4777-4850), plus f32 twins the reference
 * does not have yet: q [num_bh | batch, h_q][seq_q, d_k], k / v [num_bh | batch, h_kv][seq_k, d]; additive mask with
 * mask_bh_stride 0 (one [seq_q, seq_k] for every head) or seq_q * seq_k (one per query head). A mask slice shorter than
 * the shape reads (a slice-index panic in the reference) and h_q % h_kv != 0 are InvalidArgument. */
int32_t fth_sdpa_forward_masked_f32(const float *q, size_t q_len, const float *k, size_t k_len, const float *v, size_t v_len, size_t num_bh,
                                    size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, float scale, const float *mask, size_t mask_len,
                                    size_t mask_bh_stride, float *out, size_t out_cap);
int32_t fth_sdpa_forward_masked_f64(const double *q, size_t q_len, const double *k, size_t k_len, const double *v, size_t v_len, size_t num_bh,
                                    size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, double scale, const double *mask, size_t mask_len,
                                    size_t mask_bh_stride, double *out, size_t out_cap);
int32_t fth_sdpa_forward_masked_gqa_f32(const float *q, size_t q_len, const float *k, size_t k_len, const float *v, size_t v_len, size_t batch,
                                        size_t h_q, size_t h_kv, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, float scale,
                                        const float *mask, size_t mask_len, size_t mask_bh_stride, float *out, size_t out_cap);
int32_t fth_sdpa_forward_masked_gqa_f64(const double *q, size_t q_len, const double *k, size_t k_len, const double *v, size_t v_len, size_t batch,
                                        size_t h_q, size_t h_kv, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, double scale,
                                        const double *mask, size_t mask_len, size_t mask_bh_stride, double *out, size_t out_cap);
/* log_softmax_dim_tensor_contiguous_f32 (:39298) / _f64 (:18504): the validation of softmax_dim_tensor_contiguous.
 * cross_entropy_forward_f32 (:6717) / _f64 (:6649) -> loss [batch]; cross_entropy_backward_f32 (:6745) / _f64 (:6679)
 * -> dlogits [batch*classes]. target holds class indices (the reference's &[usize]). */
int32_t fth_log_softmax_dim_tensor_contiguous_f32(const float *input, size_t input_len, const fth_meta *meta, size_t dim, float *out,
                                                  size_t out_cap, size_t *out_len);
int32_t fth_log_softmax_dim_tensor_contiguous_f64(const double *input, size_t input_len, const fth_meta *meta, size_t dim, double *out,
                                                  size_t out_cap, size_t *out_len);
int32_t fth_cross_entropy_forward_f32(const float *logits, size_t logits_len, const uint64_t *target, size_t target_len, size_t batch,
                                      size_t classes, float *loss, size_t loss_cap);
int32_t fth_cross_entropy_forward_f64(const double *logits, size_t logits_len, const uint64_t *target, size_t target_len, size_t batch,
                                      size_t classes, double *loss, size_t loss_cap);
int32_t fth_cross_entropy_backward_f32(const float *logits, size_t logits_len, const uint64_t *target, size_t target_len, const float *dloss,
                                       size_t dloss_len, size_t batch, size_t classes, float *dlogits, size_t dlogits_cap);
int32_t fth_cross_entropy_backward_f64(const double *logits, size_t logits_len, const uint64_t *target, size_t target_len, const double *dloss,
                                       size_t dloss_len, size_t batch, size_t classes, double *dlogits, size_t dlogits_cap);
/* Backward of the fused ops on host slices. Every output has its own capacity (in elements) and must hold its result:
 * layer_norm_backward_f32 (:6189) / _f64 (:6052) -> dx [batch*norm_size], dweight, dbias [norm_size];
 * rms_norm_backward_f32 (:6574) / _f64 (:6503) -> dx, dweight (weight == NULL: no dweight, pass NULL / 0);
 * linear_backward_f64 (:17226) and the same formulas in f32 -> dx [batch*in], dweight [out*in], dbias [out] when need_bias;
 * sdpa_backward_f32 (:5539) / _f64 (:5300) -> dq, dk, dv of the shapes of q, k, v. */
int32_t fth_layer_norm_backward_f32(const float *dy, size_t dy_len, const float *x, size_t x_len, const float *weight, size_t batch,
                                    size_t norm_size, float eps, float *dx, size_t dx_cap, float *dweight, size_t dweight_cap,
                                    float *dbias, size_t dbias_cap);
int32_t fth_layer_norm_backward_f64(const double *dy, size_t dy_len, const double *x, size_t x_len, const double *weight, size_t batch,
                                    size_t norm_size, double eps, double *dx, size_t dx_cap, double *dweight, size_t dweight_cap,
                                    double *dbias, size_t dbias_cap);
int32_t fth_rms_norm_backward_f32(const float *dy, size_t dy_len, const float *x, size_t x_len, const float *weight, size_t batch,
                                  size_t norm_size, float eps, float *dx, size_t dx_cap, float *dweight, size_t dweight_cap);
int32_t fth_rms_norm_backward_f64(const double *dy, size_t dy_len, const double *x, size_t x_len, const double *weight, size_t batch,
                                  size_t norm_size, double eps, double *dx, size_t dx_cap, double *dweight, size_t dweight_cap);
int32_t fth_linear_backward_f32(const float *dy, size_t dy_len, const float *x, size_t x_len, const float *weight, size_t weight_len,
                                size_t batch, size_t in_features, size_t out_features, int32_t need_bias, float *dx, size_t dx_cap,
                                float *dweight, size_t dweight_cap, float *dbias, size_t dbias_cap);
int32_t fth_linear_backward_f64(const double *dy, size_t dy_len, const double *x, size_t x_len, const double *weight, size_t weight_len,
                                size_t batch, size_t in_features, size_t out_features, int32_t need_bias, double *dx, size_t dx_cap,
                                double *dweight, size_t dweight_cap, double *dbias, size_t dbias_cap);
int32_t fth_sdpa_backward_f32(const float *q, size_t q_len, const float *k, size_t k_len, const float *v, size_t v_len, const float *dout,
                              size_t dout_len, size_t num_bh, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, float scale,
                              int32_t causal, float *dq, size_t dq_cap, float *dk, size_t dk_cap, float *dv, size_t dv_cap);
int32_t fth_sdpa_backward_f64(const double *q, size_t q_len, const double *k, size_t k_len, const double *v, size_t v_len, const double *dout,
                              size_t dout_len, size_t num_bh, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, double scale,
                              int32_t causal, double *dq, size_t dq_cap, double *dk, size_t dk_cap, double *dv, size_t dv_cap);
/* sdpa_backward_f32_unit_dout (:5662): dOut = ones, not passed. */
int32_t fth_sdpa_backward_f32_unit_dout(const float *q, size_t q_len, const float *k, size_t k_len, const float *v, size_t v_len, size_t num_bh,
                                        size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, float scale, int32_t causal, float *dq,
                                        size_t dq_cap, float *dk, size_t dk_cap, float *dv, size_t dv_cap);
/* sdpa_backward_masked_f64 (:5423) and its f32 twin: mask slice of (num_bh - 1) * mask_bh_stride + seq_q * seq_k elements. */
int32_t fth_sdpa_backward_masked_f32(const float *q, size_t q_len, const float *k, size_t k_len, const float *v, size_t v_len, const float *dout,
                                     size_t dout_len, size_t num_bh, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, float scale,
                                     const float *mask, size_t mask_len, size_t mask_bh_stride, float *dq, size_t dq_cap, float *dk,
                                     size_t dk_cap, float *dv, size_t dv_cap);
int32_t fth_sdpa_backward_masked_f64(const double *q, size_t q_len, const double *k, size_t k_len, const double *v, size_t v_len, const double *dout,
                                     size_t dout_len, size_t num_bh, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v, double scale,
                                     const double *mask, size_t mask_len, size_t mask_bh_stride, double *dq, size_t dq_cap, double *dk,
                                     size_t dk_cap, double *dv, size_t dv_cap);
/* gelu_tensor_contiguous_f32 (:37123) / _f64 (:3657); add_tensor_contiguous_f32 (:36870) / _f64 */
int32_t fth_gelu_tensor_contiguous_f32(const float *input, size_t input_len, const fth_meta *meta,
                                       float *out, size_t out_cap, size_t *out_len);
/* The tanh form through the same validation (session op tensor_gelu_tanh behind GELU::tanh(), crates/ft-nn/src/lib.rs:1949-1957). */
int32_t fth_gelu_tanh_tensor_contiguous_f32(const float *input, size_t input_len, const fth_meta *meta, float *out, size_t out_cap,
                                            size_t *out_len);
int32_t fth_gelu_tanh_tensor_contiguous_f64(const double *input, size_t input_len, const fth_meta *meta, double *out, size_t out_cap,
                                            size_t *out_len);
int32_t fth_gelu_tensor_contiguous_f64(const double *input, size_t input_len, const fth_meta *meta,
                                       double *out, size_t out_cap, size_t *out_len);
int32_t fth_add_tensor_contiguous_f32(const float *lhs, size_t lhs_len, const float *rhs, size_t rhs_len,
                                      const fth_meta *lhs_meta, const fth_meta *rhs_meta,
                                      float *out, size_t out_cap, size_t *out_len);
int32_t fth_add_tensor_contiguous_f64(const double *lhs, size_t lhs_len, const double *rhs, size_t rhs_len,
                                      const fth_meta *lhs_meta, const fth_meta *rhs_meta,
                                      double *out, size_t out_cap, size_t *out_len);
/* transpose_2d_into_f32 (:42415) / _f64 (:42294): src [rows, cols] -> dst [cols, rows], caller buffer;
 * transpose_batched_materialize_f32 (:42526) / _f64 (:42490): src [batch, rows, cols] -> out [batch, cols, rows]. */
int32_t fth_transpose_2d_into_f32(const float *src, size_t src_len, float *dst, size_t dst_cap, size_t rows, size_t cols);
int32_t fth_transpose_2d_into_f64(const double *src, size_t src_len, double *dst, size_t dst_cap, size_t rows, size_t cols);
int32_t fth_transpose_batched_materialize_f32(const float *src, size_t src_len, size_t batch, size_t rows, size_t cols, float *out,
                                              size_t out_cap);
int32_t fth_transpose_batched_materialize_f64(const double *src, size_t src_len, size_t batch, size_t rows, size_t cols, double *out,
                                              size_t out_cap);
/* sdpa_forward_f32 (:5200) / _f64 (:4572) */
int32_t fth_sdpa_forward_f32(const float *q, size_t q_len, const float *k, size_t k_len, const float *v,
                             size_t v_len, size_t num_bh, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v,
                             float scale, int32_t causal, float *out, size_t out_cap);
int32_t fth_sdpa_forward_f64(const double *q, size_t q_len, const double *k, size_t k_len, const double *v,
                             size_t v_len, size_t num_bh, size_t seq_q, size_t seq_k, size_t d_k, size_t d_v,
                             double scale, int32_t causal, double *out, size_t out_cap);
/* index_select_tensor_contiguous_f32 (:40216) / _f64; indices are f64 values */
int32_t fth_index_select_tensor_contiguous_f32(const float *input, size_t input_len, const fth_meta *meta,
                                               size_t dim, const double *indices, size_t num_indices,
                                               float *out, size_t out_cap, size_t *out_len);
int32_t fth_index_select_tensor_contiguous_f64(const double *input, size_t input_len, const fth_meta *meta,
                                               size_t dim, const double *indices, size_t num_indices,
                                               double *out, size_t out_cap, size_t *out_len);
/* argmax_dim_tensor_contiguous_f32 (:39443) / _f64 (:18653); indices returned as float values */
int32_t fth_argmax_dim_tensor_contiguous_f32(const float *input, size_t input_len, const fth_meta *meta,
                                             size_t dim, float *out, size_t out_cap, size_t *out_len);
int32_t fth_argmax_dim_tensor_contiguous_f64(const double *input, size_t input_len, const fth_meta *meta,
                                             size_t dim, double *out, size_t out_cap, size_t *out_len);

/* ------------------------------------------------------------------------------------------ */
/* Tier B: resident tensors, stream-ordered batch, block and GPT-2-shaped runners             */
/* ------------------------------------------------------------------------------------------ */

/* GpuTensor (crates/ft-kernel-metal/src/fused.rs:540-580): a resident f32 [rows, cols] matrix. */
typedef struct fth_tensor fth_tensor;
int32_t fth_tensor_upload(const float *host, int64_t rows, int64_t cols, fth_tensor **out);
int32_t fth_tensor_alloc(int64_t rows, int64_t cols, fth_tensor **out);
int32_t fth_tensor_download(const fth_tensor *t, float *host, size_t host_cap);
int32_t fth_tensor_shape(const fth_tensor *t, int64_t *rows, int64_t *cols);
void *fth_tensor_data(const fth_tensor *t); /* device pointer */
int32_t fth_tensor_free(fth_tensor *t);
/* Bytes currently held by, and cached inside, the library's buffer pool
 * (crates/ft-core/src/buffer_pool.rs:206-329 recycles host Vecs the same way). */
int32_t fth_pool_stats(uint64_t *bytes_in_use, uint64_t *bytes_cached);
int32_t fth_pool_trim(void);

/* Batch (crates/ft-kernel-metal/src/fused.rs:676-932): every op enqueues on the batch's stream
 * and returns a fresh resident tensor; fth_batch_finish is the only synchronisation. */
typedef struct fth_batch fth_batch;
int32_t fth_batch_new(fth_batch **out);
int32_t fth_batch_free(fth_batch *b);
int32_t fth_batch_finish(fth_batch *b);
/* y = a[m,k] * w[n,k]^T (+ bias[n])  -- Batch::matmul_bias, :676-762, with the weight in the
 * [out, in] layout of ft-nn Linear (crates/ft-nn/src/lib.rs:902-1118). */
int32_t fth_batch_linear(fth_batch *b, const fth_tensor *a, const fth_tensor *w, const fth_tensor *bias, fth_tensor **out);
/* y = a[m,k] * rhs[k,n]  -- tensor_matmul layout */
int32_t fth_batch_matmul(fth_batch *b, const fth_tensor *a, const fth_tensor *rhs, fth_tensor **out);
int32_t fth_batch_layernorm(fth_batch *b, const fth_tensor *x, const fth_tensor *gamma, const fth_tensor *beta, float eps, fth_tensor **out);
int32_t fth_batch_rmsnorm(fth_batch *b, const fth_tensor *x, const fth_tensor *gamma, float eps, fth_tensor **out);
int32_t fth_batch_gelu(fth_batch *b, const fth_tensor *x, fth_tensor **out);      /* erf form, the ft-kernel-cpu arithmetic */
int32_t fth_batch_gelu_tanh(fth_batch *b, const fth_tensor *x, fth_tensor **out); /* tanh form, Batch::gelu's own (fused.rs:301-313, 814-825) */
int32_t fth_batch_add(fth_batch *b, const fth_tensor *x, const fth_tensor *y, fth_tensor **out);
int32_t fth_batch_softmax(fth_batch *b, const fth_tensor *x, fth_tensor **out);
/* Multi-head attention over [seq, d_model] q/k/v with n_heads heads (Batch::mha, :861-925);
 * `batch` sequences are stacked along rows (rows = batch * seq). */
int32_t fth_batch_mha(fth_batch *b, const fth_tensor *q, const fth_tensor *k, const fth_tensor *v,
                      int64_t n_heads, int64_t batch, int32_t causal, fth_tensor **out);

/* One layer's weights, host pointers, nn.Linear layout [out, in]
 * (LayerWeightsRef, crates/ft-kernel-metal/src/fused.rs:986-1016; topology of
 * TransformerEncoderLayer::forward_layer_masked with norm_first, crates/ft-nn/src/lib.rs:14709-14744). */
typedef struct fth_layer_weights {
    const float *ln1_w, *ln1_b;     /* [d_model] */
    const float *wq, *bq;           /* [d_model, d_model], [d_model] */
    const float *wk, *bk;
    const float *wv, *bv;
    const float *wo, *bo;
    const float *ln2_w, *ln2_b;
    const float *w1, *b1;           /* [d_ff, d_model], [d_ff] */
    const float *w2, *b2;           /* [d_model, d_ff], [d_model] */
} fth_layer_weights;

/* EncoderGpu (crates/ft-kernel-metal/src/fused.rs:1024-1190): weights uploaded once; forward
 * runs `n_layers` pre-LN blocks on a resident [batch*seq, d_model] activation. */
typedef struct fth_encoder fth_encoder;
int32_t fth_encoder_new(int64_t d_model, int64_t n_heads, int64_t d_ff, float ln_eps, int32_t causal,
                        const fth_layer_weights *layers, int64_t n_layers, fth_encoder **out);
int32_t fth_encoder_free(fth_encoder *e);
/* Feed-forward activation of the blocks: the erf form of ft-kernel-cpu (default) or the tanh form the reference's
 * Metal encoder computes (crates/ft-kernel-metal/src/fused.rs:301-313) and GPT-2 checkpoints were trained with.
 * Refused once a graph of this encoder has been captured. */
enum { FTH_ACT_GELU_ERF = 0, FTH_ACT_GELU_TANH = 1 };
int32_t fth_encoder_set_activation(fth_encoder *e, int32_t activation);
/* Host in / host out (EncoderGpu::forward, :1136-1146). */
int32_t fth_encoder_forward(fth_encoder *e, const float *input, int64_t batch, int64_t seq, float *out, size_t out_cap);
/* Resident in / resident out on stream `s`; no synchronisation. `x` [batch*seq, d_model]. */
int32_t fth_encoder_forward_dev(fth_encoder *e, const float *x_dev, int64_t batch, int64_t seq, float *out_dev, fth_stream s);
/* Captures forward_dev for (x_dev, out_dev, batch, seq, s) into a HIP graph and replays it: one
 * launch per forward. The graph holds device addresses: the caller's two buffers must stay valid
 * while the encoder lives; the encoder's activations and the stream's GEMM split-tile workspace it
 * also records are never released before fth_encoder_free. Returns FTH_ERR_UNAVAILABLE while a
 * rocprofiler tool library is loaded in the process (trace the eager entry point instead). */
int32_t fth_encoder_forward_graph(fth_encoder *e, const float *x_dev, int64_t batch, int64_t seq, float *out_dev, fth_stream s);

/* ------------------------------------------------------------------------------------------ */
/* Weight ingestion: safetensors -> resident buffers                                           */
/* ------------------------------------------------------------------------------------------ */
/* load_safetensors (crates/ft-serialize/src/lib.rs:2170-2176), load_safetensors_from_bytes (:2179-2241) and
 * load_safetensors_metadata (:2274-2286), for a caller whose tensors live on the GPU. open / open_bytes validate the
 * whole container (the checks of safetensors 0.8.0's SafeTensors::deserialize, then the loader's own: only F64 / F32 /
 * F16 / BF16 tensors, each of exactly numel * width bytes) and fail with FTH_ERR_CORRUPT where the reference returns
 * TensorIOError::Corrupt, FTH_ERR_IO where it returns TensorIOError::Io. The file is memory-mapped; `open_bytes` borrows
 * `data`, which must outlive the handle. Tensors are listed in name order (the reference's BTreeMap). */
typedef struct fth_safetensors fth_safetensors;
typedef struct fth_safetensors_tensor {
    int32_t dtype; /* FTH_DTYPE_* as stored in the file */
    int32_t ndim;
    uint64_t shape[FTH_MAX_DIMS];
    uint64_t numel;
    uint64_t byte_len;
} fth_safetensors_tensor;
int32_t fth_safetensors_open(const char *path, fth_safetensors **out);
int32_t fth_safetensors_open_bytes(const void *data, size_t len, fth_safetensors **out);
int32_t fth_safetensors_close(fth_safetensors *f);
int64_t fth_safetensors_count(const fth_safetensors *f);
const char *fth_safetensors_name(const fth_safetensors *f, int64_t index); /* NULL past the end */
int32_t fth_safetensors_info(const fth_safetensors *f, const char *name, fth_safetensors_tensor *info);
/* The tensor's little-endian bytes as stored (what the reference decodes into a DenseTensor), into host memory. */
int32_t fth_safetensors_read(const fth_safetensors *f, const char *name, void *dst, size_t dst_bytes);
/* The tensor into device memory as f32 / f64, whatever its stored type (F16 / BF16 / F32 widen exactly; F64 -> f32
 * rounds to nearest), optionally transposed when it is a matrix ([rows, cols] in the file -> [cols, rows] in dst; GPT-2
 * checkpoints store their projections [in, out], the linear kernels read [out, in]). The bytes go through pinned staging
 * buffers with asynchronous copies and are converted / transposed on the GPU. Synchronises `s` before returning. */
int32_t fth_safetensors_read_f32_dev(const fth_safetensors *f, const char *name, int32_t transpose_2d, float *dst_dev, size_t dst_elems,
                                     fth_stream s);
int32_t fth_safetensors_read_f64_dev(const fth_safetensors *f, const char *name, int32_t transpose_2d, double *dst_dev, size_t dst_elems,
                                     fth_stream s);
/* The "__metadata__" string map: number of entries (-1 if the file has none) and lookup (NULL if absent). */
int32_t fth_safetensors_metadata_count(const fth_safetensors *f);
const char *fth_safetensors_metadata(const fth_safetensors *f, const char *key);

/* The reference's NATIVE state-dict container, load_state_dict (crates/ft-serialize/src/lib.rs:996-1002) and
 * load_state_dict_from_bytes (:1005-1160), through the same kind of handle: "FTSV", version u32 (<= 1), tensor count u64,
 * then per tensor key length u64, key, ndim u64, u64 dims, dtype tag u8 (0 F64, 1 F32, 2 F16, 3 BF16) and the payload,
 * all little-endian (written by write_state_dict_to_writer :786-860). open / open_bytes validate the whole container in
 * the reference's order and fail as it does: FTH_ERR_INVALID_MAGIC, FTH_ERR_UNSUPPORTED_VERSION, and FTH_ERR_CORRUPT with
 * the reference's reason text (truncated key / shape / dtype / payload, duplicate key, a tensor count or byte count the
 * file cannot hold, trailing bytes). One deviation: a key that contains a NUL byte, which the reference accepts, cannot be
 * named through a C string and makes open fail with FTH_ERR_CORRUPT. Listing (name order), info and the host and device
 * reads behave as for safetensors; there is no metadata map. */
typedef struct fth_safetensors fth_statedict;
int32_t fth_statedict_open(const char *path, fth_statedict **out);
int32_t fth_statedict_open_bytes(const void *data, size_t len, fth_statedict **out);
int32_t fth_statedict_close(fth_statedict *f);
int64_t fth_statedict_count(const fth_statedict *f);
const char *fth_statedict_name(const fth_statedict *f, int64_t index);
int32_t fth_statedict_info(const fth_statedict *f, const char *name, fth_safetensors_tensor *info);
int32_t fth_statedict_read(const fth_statedict *f, const char *name, void *dst, size_t dst_bytes);
int32_t fth_statedict_read_f32_dev(const fth_statedict *f, const char *name, int32_t transpose_2d, float *dst_dev, size_t dst_elems,
                                   fth_stream s);
int32_t fth_statedict_read_f64_dev(const fth_statedict *f, const char *name, int32_t transpose_2d, double *dst_dev, size_t dst_elems,
                                   fth_stream s);

/* GPT-2-shaped decoder: learned positions, pre-LN blocks, final LN, LM head tied to wte. */
typedef struct fth_gpt2 fth_gpt2;
int32_t fth_gpt2_new(int64_t vocab, int64_t max_pos, int64_t d_model, int64_t n_heads, int64_t d_ff, float ln_eps,
                     const float *wte, const float *wpe, const fth_layer_weights *layers, int64_t n_layers,
                     const float *lnf_w, const float *lnf_b, fth_gpt2 **out);
/* The same model with its weights read from a GPT-2 checkpoint in safetensors form, straight into resident buffers:
 * "wte.weight" [vocab, d], "wpe.weight" [max_pos, d], per layer i "h.i.ln_1.{weight,bias}", "h.i.attn.c_attn.{weight [d, 3d],
 * bias}", "h.i.attn.c_proj.{weight [d, d], bias}", "h.i.ln_2.{weight,bias}", "h.i.mlp.c_fc.{weight [d, d_ff], bias}",
 * "h.i.mlp.c_proj.{weight [d_ff, d], bias}", "ln_f.{weight,bias}", each optionally under a "transformer." prefix. The
 * projection matrices are stored [in, out] and are transposed on the GPU while loading; F16 / BF16 / F64 tensors are
 * converted to f32 there. Shapes are taken from the file; other tensors in it (attention mask buffers) are ignored.
 * A missing or mis-shaped tensor is FTH_ERR_CORRUPT. activation: FTH_ACT_GELU_TANH is what GPT-2 was trained with. */
int32_t fth_gpt2_from_safetensors(const fth_safetensors *f, int64_t n_heads, float ln_eps, int32_t activation, fth_gpt2 **out);
/* The same from a native state-dict container holding the same tensor names. */
int32_t fth_gpt2_from_statedict(const fth_statedict *f, int64_t n_heads, float ln_eps, int32_t activation, fth_gpt2 **out);
/* vocab, max_pos, d_model, n_heads, d_ff, n_layers of a model (any pointer may be NULL). */
int32_t fth_gpt2_dims(const fth_gpt2 *g, int64_t *vocab, int64_t *max_pos, int64_t *d_model, int64_t *n_heads, int64_t *d_ff,
                      int64_t *n_layers);
int32_t fth_gpt2_free(fth_gpt2 *g);
int32_t fth_gpt2_set_activation(fth_gpt2 *g, int32_t activation); /* FTH_ACT_GELU_ERF (default) | FTH_ACT_GELU_TANH */
/* ids: device f64 token-id values [batch*seq] (indices are float-valued tensors in the reference,
 * crates/ft-nn/examples/bert_rerank_spike.rs:61-63). logits_dev [batch*seq, vocab] and
 * argmax_dev [batch*seq] (f32 index values) may each be NULL to skip that output; when logits_dev
 * is NULL and argmax_dev is not, logits go to an internal buffer. */
int32_t fth_gpt2_forward_dev(fth_gpt2 *g, const double *ids_dev, int64_t batch, int64_t seq,
                             float *logits_dev, float *argmax_dev, fth_stream s);
/* Final hidden state [batch*seq, d_model] of the last forward (device pointer, valid until the next). */
const float *fth_gpt2_hidden_dev(const fth_gpt2 *g);
/* Position of the first token id of the last forward that failed normalize_strict_index_value
 * (crates/ft-kernel-cpu/src/lib.rs:20058-20090), or -1. Synchronises. The reference returns
 * InvalidDimension for such an id; here the affected rows of the embedding are left unwritten and
 * the caller checks this after the forward. */
int32_t fth_gpt2_bad_index(const fth_gpt2 *g, int64_t *position);

#ifdef __cplusplus
}
#endif
#endif /* FT_KERNEL_HIP_H */
