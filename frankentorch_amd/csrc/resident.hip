// Tier B of the C ABI: resident tensors, a stream-ordered batch of ops, and the pre-LN block /
// GPT-2-shaped runners that keep every activation in HBM between kernels. Modelled on
// ft_kernel_metal::fused::{GpuTensor, Batch, EncoderGpu} (crates/ft-kernel-metal/src/fused.rs:
// 540-933, 986-1190), with the arithmetic of ft-kernel-cpu (erf GELU, fp32 operands) rather than
// Metal's (tanh GELU, f16-staged tiles).
//
// Block topology (TransformerEncoderLayer::forward_layer_masked with norm_first,
// crates/ft-nn/src/lib.rs:14709-14744; MultiheadAttention::forward_qkv_masked, :5088-5198):
//   h   = LN1(x)
//   qkv = h . [Wq; Wk; Wv]^T + [bq; bk; bv]          one GEMM, N = 3 * d_model
//   ctx = SDPA(q, k, v)                              reads the packed qkv rows head by head and
//                                                    writes [tokens, d_model]: no permuted copies
//   x1  = (ctx . Wo^T + bo) + x                      bias and residual in the GEMM epilogue
//   h2  = LN2(x1)
//   f   = gelu(h2 . W1^T + b1)                       bias and GELU in the epilogue
//   x2  = (f . W2^T + b2) + x1
// Every epilogue step keeps its own rounding, so the result is what the unfused op sequence
// would give with the same GEMM.

#include <cmath>
#include <cstdlib>
#include <map>
#include <mutex>
#include <new>
#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

#include "common.hpp"
#include "pool.hpp"

// ---------------------------------------------------------------------------------------------
// Pool
// ---------------------------------------------------------------------------------------------
namespace fth {
namespace {
struct Pool {
    std::mutex mu;
    std::multimap<size_t, void *> free_blocks;      // size class -> cached block
    std::unordered_map<void *, size_t> live;        // block -> size class
    uint64_t in_use = 0, cached = 0;
};
Pool &pool() {
    static Pool *p = new Pool();  // never destroyed: HIP may already be torn down at exit
    return *p;
}
size_t size_class(size_t bytes) {
    const size_t g = bytes < (1u << 20) ? 512 : (1u << 20);
    return (bytes + g - 1) / g * g;
}
int32_t trim_locked(Pool &p) {
    for (auto &kv : p.free_blocks) (void)hipFree(kv.second);
    p.free_blocks.clear();
    p.cached = 0;
    return FTH_OK;
}
}  // namespace

int32_t pool_alloc(void **dptr, size_t bytes) {
    *dptr = nullptr;
    if (bytes == 0) return FTH_OK;
    FTH_REQUIRE_DEVICE();
    const size_t cls = size_class(bytes);
    Pool &p = pool();
    std::lock_guard<std::mutex> lock(p.mu);
    auto it = p.free_blocks.find(cls);
    void *ptr = nullptr;
    if (it != p.free_blocks.end()) {
        ptr = it->second;
        p.free_blocks.erase(it);
        p.cached -= cls;
    } else {
        hipError_t e = hipMalloc(&ptr, cls);
        if (e == hipErrorOutOfMemory) {
            (void)hipGetLastError();
            // Cached blocks may still be in use by queued kernels: drain before releasing them.
            (void)hipDeviceSynchronize();
            trim_locked(p);
            e = hipMalloc(&ptr, cls);
        }
        if (e != hipSuccess) return hip_fail(e, "hipMalloc");
    }
    p.live[ptr] = cls;
    p.in_use += cls;
    *dptr = ptr;
    return FTH_OK;
}

void pool_free(void *dptr) {
    if (!dptr) return;
    Pool &p = pool();
    std::lock_guard<std::mutex> lock(p.mu);
    auto it = p.live.find(dptr);
    if (it == p.live.end()) return;
    const size_t cls = it->second;
    p.live.erase(it);
    p.in_use -= cls;
    p.free_blocks.emplace(cls, dptr);
    p.cached += cls;
}

void pool_stats(uint64_t *in_use, uint64_t *cached) {
    Pool &p = pool();
    std::lock_guard<std::mutex> lock(p.mu);
    if (in_use) *in_use = p.in_use;
    if (cached) *cached = p.cached;
}

int32_t pool_trim() {
    if (!available()) return FTH_OK;
    Pool &p = pool();
    (void)hipDeviceSynchronize();
    std::lock_guard<std::mutex> lock(p.mu);
    return trim_locked(p);
}

Scratch::~Scratch() {
    for (int i = 0; i < n_; ++i) pool_free(ptrs_[i]);
}
int32_t Scratch::get(void **dptr, size_t bytes) {
    if (n_ >= kMax) return set_error(FTH_ERR_KERNEL, "scratch list full");
    int32_t rc = pool_alloc(dptr, bytes);
    if (rc == FTH_OK && *dptr) ptrs_[n_++] = *dptr;
    return rc;
}
}  // namespace fth

// ---------------------------------------------------------------------------------------------
// Resident tensors and the batch
// ---------------------------------------------------------------------------------------------
struct fth_tensor {
    float *data;
    int64_t rows, cols;
};
struct fth_batch {
    int64_t ops;
};

namespace {

int32_t tensor_new(int64_t rows, int64_t cols, fth_tensor **out) {
    FTH_ARG(out != nullptr, "tensor: out is NULL");
    *out = nullptr;
    FTH_ARG(rows >= 0 && cols >= 0, "tensor: negative extent");
    int64_t n;
    if (__builtin_mul_overflow(rows, cols, &n) || n > (int64_t)(1ull << 60))
        return fth::set_error(FTH_ERR_SIZE_OVERFLOW, "tensor: %lld x %lld overflows", (long long)rows, (long long)cols);
    FTH_REQUIRE_DEVICE();
    void *p = nullptr;
    if (int32_t rc = fth::pool_alloc(&p, (size_t)n * sizeof(float))) return rc;
    fth_tensor *t = new (std::nothrow) fth_tensor{static_cast<float *>(p), rows, cols};
    if (!t) {
        fth::pool_free(p);
        return fth::set_error(FTH_ERR_KERNEL, "tensor: host allocation failed");
    }
    *out = t;
    return FTH_OK;
}

fth_gemm_desc linear_desc(int64_t m, int64_t n, int64_t k, int epi) {
    fth_gemm_desc d{};
    d.m = m; d.n = n; d.k = k;
    d.lda = k; d.ldb = k; d.ldc = n;
    d.batch = 1;
    d.stride_a = d.stride_b = d.stride_c = 0;
    d.trans_b = 1;
    d.epilogue = epi;
    return d;
}

// Device copy of one layer's weights, QKV packed as one [3d, d] matrix.
struct LayerDev {
    float *ln1_w, *ln1_b, *wqkv, *bqkv, *wo, *bo, *ln2_w, *ln2_b, *w1, *b1, *w2, *b2;
};

struct Workspace {
    int64_t tokens = 0;
    float *h = nullptr, *qkv = nullptr, *ctx = nullptr, *xa = nullptr, *xb = nullptr, *ff = nullptr;
};

struct Stack {
    int64_t d_model = 0, n_heads = 0, d_ff = 0;
    float eps = 1e-5f;
    int causal = 1;
    int gelu_epilogue = FTH_EPI_GELU;  // FTH_EPI_GELU (erf form) or FTH_EPI_GELU_TANH
    std::vector<LayerDev> layers;
    std::vector<void *> owned;  // every device block this stack allocated
    Workspace ws;
    std::mutex mu;

    ~Stack() {
        for (void *p : owned) fth::pool_free(p);
    }
    int32_t upload(const float *host, int64_t n, float **dev) {
        void *p = nullptr;
        if (int32_t rc = fth::pool_alloc(&p, (size_t)n * sizeof(float))) return rc;
        owned.push_back(p);
        *dev = static_cast<float *>(p);
        if (n) FTH_HIP(hipMemcpy(p, host, (size_t)n * sizeof(float), hipMemcpyHostToDevice));
        return FTH_OK;
    }
    int32_t fill(float v, int64_t n, float **dev) {
        std::vector<float> tmp((size_t)n, v);
        return upload(tmp.data(), n, dev);
    }
    int32_t add_layer(const fth_layer_weights &w) {
        const int64_t d = d_model, f = d_ff;
        FTH_ARG(w.wq && w.wk && w.wv && w.wo && w.w1 && w.w2, "layer: a projection weight is NULL");
        LayerDev L = {};
        // Optional affine / bias vectors default to the identity (gamma 1, beta / bias 0).
        int32_t rc;
        if ((rc = w.ln1_w ? upload(w.ln1_w, d, &L.ln1_w) : fill(1.f, d, &L.ln1_w))) return rc;
        if ((rc = w.ln1_b ? upload(w.ln1_b, d, &L.ln1_b) : fill(0.f, d, &L.ln1_b))) return rc;
        if ((rc = w.ln2_w ? upload(w.ln2_w, d, &L.ln2_w) : fill(1.f, d, &L.ln2_w))) return rc;
        if ((rc = w.ln2_b ? upload(w.ln2_b, d, &L.ln2_b) : fill(0.f, d, &L.ln2_b))) return rc;
        std::vector<float> pack((size_t)(3 * d * d)), bpack((size_t)(3 * d), 0.f);
        std::memcpy(pack.data(), w.wq, sizeof(float) * d * d);
        std::memcpy(pack.data() + d * d, w.wk, sizeof(float) * d * d);
        std::memcpy(pack.data() + 2 * d * d, w.wv, sizeof(float) * d * d);
        if (w.bq) std::memcpy(bpack.data(), w.bq, sizeof(float) * d);
        if (w.bk) std::memcpy(bpack.data() + d, w.bk, sizeof(float) * d);
        if (w.bv) std::memcpy(bpack.data() + 2 * d, w.bv, sizeof(float) * d);
        if ((rc = upload(pack.data(), 3 * d * d, &L.wqkv))) return rc;
        if ((rc = upload(bpack.data(), 3 * d, &L.bqkv))) return rc;
        if ((rc = upload(w.wo, d * d, &L.wo))) return rc;
        if ((rc = w.bo ? upload(w.bo, d, &L.bo) : fill(0.f, d, &L.bo))) return rc;
        if ((rc = upload(w.w1, f * d, &L.w1))) return rc;
        if ((rc = w.b1 ? upload(w.b1, f, &L.b1) : fill(0.f, f, &L.b1))) return rc;
        if ((rc = upload(w.w2, d * f, &L.w2))) return rc;
        if ((rc = w.b2 ? upload(w.b2, d, &L.b2) : fill(0.f, d, &L.b2))) return rc;
        layers.push_back(L);
        return FTH_OK;
    }
    int32_t ensure_workspace(int64_t tokens) {
        if (tokens <= ws.tokens) return FTH_OK;
        // Pending kernels may still use the old blocks; they are recycled only through the pool,
        // and every user of this stack launches on a stream ordered after them.
        const int64_t d = d_model;
        struct Req { float **p; int64_t n; } reqs[] = {
            {&ws.h, tokens * d}, {&ws.qkv, tokens * 3 * d}, {&ws.ctx, tokens * d},
            {&ws.xa, tokens * d}, {&ws.xb, tokens * d}, {&ws.ff, tokens * d_ff}};
        for (auto &r : reqs) {
            void *p = nullptr;
            if (int32_t rc = fth::pool_alloc(&p, (size_t)r.n * sizeof(float))) return rc;
            owned.push_back(p);
            *r.p = static_cast<float *>(p);
        }
        ws.tokens = tokens;
        return FTH_OK;
    }
    // Runs every layer: reads x_in, leaves the result in *x_out (one of the workspace buffers,
    // or `final_out` when given).
    int32_t run(const float *x_in, int64_t batch, int64_t seq, float *final_out, const float **x_out, fth_stream s) {
        const int64_t T = batch * seq, d = d_model, hd = d / n_heads;
        if (int32_t rc = ensure_workspace(T)) return rc;
        const float *x = x_in;
        const float scale = (float)(1.0 / std::sqrt((double)hd));
        for (size_t li = 0; li < layers.size(); ++li) {
            const LayerDev &L = layers[li];
            const bool last = li + 1 == layers.size();
            int32_t rc;
            if ((rc = fth_dev_layer_norm_f32(x, L.ln1_w, L.ln1_b, ws.h, T, d, eps, s))) return rc;
            fth_gemm_desc g = linear_desc(T, 3 * d, d, FTH_EPI_BIAS);
            if ((rc = fth_dev_gemm_f32(&g, 1.f, ws.h, L.wqkv, ws.qkv, L.bqkv, nullptr, s))) return rc;
            fth_sdpa_desc a;
            a.num_bh = batch * n_heads; a.heads = n_heads;
            a.seq_q = seq; a.seq_k = seq; a.d_k = hd; a.d_v = hd;
            a.q_batch_stride = a.k_batch_stride = a.v_batch_stride = seq * 3 * d;
            a.q_head_stride = a.k_head_stride = a.v_head_stride = hd;
            a.q_row_stride = a.k_row_stride = a.v_row_stride = 3 * d;
            a.o_batch_stride = seq * d; a.o_head_stride = hd; a.o_row_stride = d;
            a.causal = causal; a.kv_group = 0;
            if ((rc = fth_dev_sdpa_forward_f32(&a, scale, ws.qkv, ws.qkv + d, ws.qkv + 2 * d, ws.ctx, s))) return rc;
            g = linear_desc(T, d, d, FTH_EPI_BIAS | FTH_EPI_RESIDUAL);
            if ((rc = fth_dev_gemm_f32(&g, 1.f, ws.ctx, L.wo, ws.xa, L.bo, x, s))) return rc;
            if ((rc = fth_dev_layer_norm_f32(ws.xa, L.ln2_w, L.ln2_b, ws.h, T, d, eps, s))) return rc;
            g = linear_desc(T, d_ff, d, FTH_EPI_BIAS | gelu_epilogue);
            if ((rc = fth_dev_gemm_f32(&g, 1.f, ws.h, L.w1, ws.ff, L.b1, nullptr, s))) return rc;
            float *dst = (last && final_out) ? final_out : ws.xb;
            g = linear_desc(T, d, d_ff, FTH_EPI_BIAS | FTH_EPI_RESIDUAL);
            if ((rc = fth_dev_gemm_f32(&g, 1.f, ws.ff, L.w2, dst, L.b2, ws.xa, s))) return rc;
            // The next layer reads xb as its input and residual while it writes xa, and only
            // overwrites xb in its last GEMM, which no longer reads it.
            x = dst;
        }
        if (layers.empty() && final_out) {
            FTH_HIP(hipMemcpyAsync(final_out, x_in, (size_t)T * d * sizeof(float), hipMemcpyDeviceToDevice, fth::resolve_stream(s)));
            x = final_out;
        }
        if (x_out) *x_out = x;
        return FTH_OK;
    }
};

int32_t check_dims(int64_t d_model, int64_t n_heads, int64_t d_ff, int64_t n_layers) {
    FTH_ARG(d_model > 0 && n_heads > 0 && d_ff > 0 && n_layers >= 0, "non-positive model dimension");
    FTH_ARG(d_model % n_heads == 0, "d_model %lld is not divisible by n_heads %lld", (long long)d_model, (long long)n_heads);
    return FTH_OK;
}

// True when the process runs under a rocprofiler tool (rocprofv3 exports ROCP_TOOL_LIBRARIES and
// preloads its tool library).
bool profiler_tool_loaded() {
    static const bool v = [] {
        const char *tool = std::getenv("ROCP_TOOL_LIBRARIES");
        if (tool && *tool) return true;
        const char *pre = std::getenv("LD_PRELOAD");
        return pre && std::strstr(pre, "rocprofiler") != nullptr;
    }();
    return v;
}

struct GraphKey {
    const void *x, *out;
    int64_t batch, seq;
    fth_stream s;
    bool operator<(const GraphKey &o) const {
        return std::tie(x, out, batch, seq, s) < std::tie(o.x, o.out, o.batch, o.seq, o.s);
    }
};

}  // namespace

struct fth_encoder {
    Stack stack;
    std::map<GraphKey, hipGraphExec_t> graphs;
    std::vector<hipGraph_t> graph_templates;
};

struct fth_gpt2 {
    Stack stack;
    int64_t vocab = 0, max_pos = 0;
    float *wte = nullptr, *wpe = nullptr, *lnf_w = nullptr, *lnf_b = nullptr;
    float *x0 = nullptr, *hidden = nullptr, *logits = nullptr, *group_max = nullptr;
    int64_t *bad = nullptr;
    int64_t tokens_cap = 0, logits_cap = 0, group_max_cap = 0;
};

extern "C" {

int32_t fth_tensor_upload(const float *host, int64_t rows, int64_t cols, fth_tensor **out) {
    if (int32_t rc = tensor_new(rows, cols, out)) return rc;
    const size_t bytes = (size_t)rows * (size_t)cols * sizeof(float);
    if (bytes) {
        if (!host) {
            fth_tensor_free(*out);
            *out = nullptr;
            return fth::set_error(FTH_ERR_INVALID_ARGUMENT, "tensor_upload: host is NULL");
        }
        hipError_t e = hipMemcpy((*out)->data, host, bytes, hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            fth_tensor_free(*out);
            *out = nullptr;
            return fth::hip_fail(e, "hipMemcpy(H2D)");
        }
    }
    return FTH_OK;
}

int32_t fth_tensor_alloc(int64_t rows, int64_t cols, fth_tensor **out) { return tensor_new(rows, cols, out); }

int32_t fth_tensor_download(const fth_tensor *t, float *host, size_t host_cap) {
    FTH_ARG(t != nullptr, "tensor_download: tensor is NULL");
    const size_t n = (size_t)t->rows * (size_t)t->cols;
    if (host_cap < n || (n && !host))
        return fth::set_error(FTH_ERR_OUTPUT_TOO_SMALL, "tensor_download: buffer holds %zu elements, tensor has %zu", host_cap, n);
    FTH_REQUIRE_DEVICE();
    // Ops queued on the library stream finish first: hipMemcpy orders after blocking streams.
    if (n) FTH_HIP(hipMemcpy(host, t->data, n * sizeof(float), hipMemcpyDeviceToHost));
    return FTH_OK;
}

int32_t fth_tensor_shape(const fth_tensor *t, int64_t *rows, int64_t *cols) {
    FTH_ARG(t != nullptr, "tensor_shape: tensor is NULL");
    if (rows) *rows = t->rows;
    if (cols) *cols = t->cols;
    return FTH_OK;
}

void *fth_tensor_data(const fth_tensor *t) { return t ? t->data : nullptr; }

int32_t fth_tensor_free(fth_tensor *t) {
    if (!t) return FTH_OK;
    fth::pool_free(t->data);
    delete t;
    return FTH_OK;
}

int32_t fth_pool_stats(uint64_t *bytes_in_use, uint64_t *bytes_cached) {
    fth::pool_stats(bytes_in_use, bytes_cached);
    return FTH_OK;
}
int32_t fth_pool_trim(void) { return fth::pool_trim(); }

int32_t fth_batch_new(fth_batch **out) {
    FTH_ARG(out != nullptr, "batch_new: out is NULL");
    *out = nullptr;
    FTH_REQUIRE_DEVICE();
    *out = new (std::nothrow) fth_batch{0};
    if (!*out) return fth::set_error(FTH_ERR_KERNEL, "batch_new: host allocation failed");
    return FTH_OK;
}
int32_t fth_batch_free(fth_batch *b) {
    delete b;
    return FTH_OK;
}
int32_t fth_batch_finish(fth_batch *b) {
    FTH_ARG(b != nullptr, "batch_finish: batch is NULL");
    return fth_stream_synchronize(nullptr);
}

#define FTH_BATCH_PROLOGUE(name)                       \
    FTH_ARG(b != nullptr && out != nullptr, name ": NULL batch or out"); \
    *out = nullptr;                                    \
    b->ops++;

static int32_t finish_op(int32_t rc, fth_tensor *t, fth_tensor **out) {
    if (rc) {
        fth_tensor_free(t);
        return rc;
    }
    *out = t;
    return FTH_OK;
}

int32_t fth_batch_linear(fth_batch *b, const fth_tensor *a, const fth_tensor *w, const fth_tensor *bias, fth_tensor **out) {
    FTH_BATCH_PROLOGUE("batch_linear");
    FTH_ARG(a && w, "batch_linear: NULL operand");
    FTH_ARG(a->cols == w->cols, "batch_linear: a is [%lld,%lld] but w is [%lld,%lld]", (long long)a->rows,
            (long long)a->cols, (long long)w->rows, (long long)w->cols);
    FTH_ARG(!bias || bias->rows * bias->cols == w->rows, "batch_linear: bias length != out features");
    fth_tensor *t;
    if (int32_t rc = tensor_new(a->rows, w->rows, &t)) return rc;
    fth_gemm_desc g = linear_desc(a->rows, w->rows, a->cols, bias ? FTH_EPI_BIAS : FTH_EPI_NONE);
    return finish_op(fth_dev_gemm_f32(&g, 1.f, a->data, w->data, t->data, bias ? bias->data : nullptr, nullptr, nullptr), t, out);
}

int32_t fth_batch_matmul(fth_batch *b, const fth_tensor *a, const fth_tensor *rhs, fth_tensor **out) {
    FTH_BATCH_PROLOGUE("batch_matmul");
    FTH_ARG(a && rhs, "batch_matmul: NULL operand");
    FTH_ARG(a->cols == rhs->rows, "batch_matmul: inner dimensions differ (%lld vs %lld)", (long long)a->cols, (long long)rhs->rows);
    fth_tensor *t;
    if (int32_t rc = tensor_new(a->rows, rhs->cols, &t)) return rc;
    fth_gemm_desc g = linear_desc(a->rows, rhs->cols, a->cols, FTH_EPI_NONE);
    g.trans_b = 0;
    g.ldb = rhs->cols;
    return finish_op(fth_dev_gemm_f32(&g, 1.f, a->data, rhs->data, t->data, nullptr, nullptr, nullptr), t, out);
}

int32_t fth_batch_layernorm(fth_batch *b, const fth_tensor *x, const fth_tensor *gamma, const fth_tensor *beta, float eps, fth_tensor **out) {
    FTH_BATCH_PROLOGUE("batch_layernorm");
    FTH_ARG(x != nullptr, "batch_layernorm: NULL operand");
    FTH_ARG((!gamma || gamma->rows * gamma->cols == x->cols) && (!beta || beta->rows * beta->cols == x->cols),
            "batch_layernorm: gamma/beta length != cols");
    fth_tensor *t;
    if (int32_t rc = tensor_new(x->rows, x->cols, &t)) return rc;
    return finish_op(fth_dev_layer_norm_f32(x->data, gamma ? gamma->data : nullptr, beta ? beta->data : nullptr, t->data,
                                            x->rows, x->cols, eps, nullptr), t, out);
}

int32_t fth_batch_rmsnorm(fth_batch *b, const fth_tensor *x, const fth_tensor *gamma, float eps, fth_tensor **out) {
    FTH_BATCH_PROLOGUE("batch_rmsnorm");
    FTH_ARG(x != nullptr, "batch_rmsnorm: NULL operand");
    FTH_ARG(!gamma || gamma->rows * gamma->cols == x->cols, "batch_rmsnorm: gamma length != cols");
    fth_tensor *t;
    if (int32_t rc = tensor_new(x->rows, x->cols, &t)) return rc;
    return finish_op(fth_dev_rms_norm_f32(x->data, gamma ? gamma->data : nullptr, t->data, x->rows, x->cols, eps, nullptr), t, out);
}

int32_t fth_batch_gelu_tanh(fth_batch *b, const fth_tensor *x, fth_tensor **out) {
    FTH_BATCH_PROLOGUE("batch_gelu_tanh");
    FTH_ARG(x != nullptr, "batch_gelu_tanh: NULL operand");
    fth_tensor *t;
    if (int32_t rc = tensor_new(x->rows, x->cols, &t)) return rc;
    return finish_op(fth_dev_gelu_tanh_f32(x->data, t->data, x->rows * x->cols, nullptr), t, out);
}

int32_t fth_batch_gelu(fth_batch *b, const fth_tensor *x, fth_tensor **out) {
    FTH_BATCH_PROLOGUE("batch_gelu");
    FTH_ARG(x != nullptr, "batch_gelu: NULL operand");
    fth_tensor *t;
    if (int32_t rc = tensor_new(x->rows, x->cols, &t)) return rc;
    return finish_op(fth_dev_gelu_f32(x->data, t->data, x->rows * x->cols, nullptr), t, out);
}

int32_t fth_batch_add(fth_batch *b, const fth_tensor *x, const fth_tensor *y, fth_tensor **out) {
    FTH_BATCH_PROLOGUE("batch_add");
    FTH_ARG(x && y, "batch_add: NULL operand");
    FTH_ARG(x->rows == y->rows && x->cols == y->cols, "batch_add: shapes differ");
    fth_tensor *t;
    if (int32_t rc = tensor_new(x->rows, x->cols, &t)) return rc;
    return finish_op(fth_dev_add_f32(x->data, y->data, t->data, x->rows * x->cols, nullptr), t, out);
}

int32_t fth_batch_softmax(fth_batch *b, const fth_tensor *x, fth_tensor **out) {
    FTH_BATCH_PROLOGUE("batch_softmax");
    FTH_ARG(x != nullptr, "batch_softmax: NULL operand");
    fth_tensor *t;
    if (int32_t rc = tensor_new(x->rows, x->cols, &t)) return rc;
    return finish_op(fth_dev_softmax_lastdim_f32(x->data, t->data, x->rows, x->cols, nullptr), t, out);
}

int32_t fth_batch_mha(fth_batch *b, const fth_tensor *q, const fth_tensor *k, const fth_tensor *v, int64_t n_heads,
                      int64_t batch, int32_t causal, fth_tensor **out) {
    FTH_BATCH_PROLOGUE("batch_mha");
    FTH_ARG(q && k && v, "batch_mha: NULL operand");
    FTH_ARG(n_heads > 0 && batch > 0, "batch_mha: n_heads and batch must be positive");
    const int64_t d = q->cols;
    FTH_ARG(k->cols == d && v->cols == d && d % n_heads == 0, "batch_mha: d_model mismatch or not divisible by heads");
    FTH_ARG(q->rows % batch == 0 && k->rows % batch == 0 && k->rows == v->rows, "batch_mha: rows not divisible by batch");
    const int64_t sq = q->rows / batch, sk = k->rows / batch, hd = d / n_heads;
    fth_tensor *t;
    if (int32_t rc = tensor_new(q->rows, d, &t)) return rc;
    fth_sdpa_desc a;
    a.num_bh = batch * n_heads; a.heads = n_heads;
    a.seq_q = sq; a.seq_k = sk; a.d_k = hd; a.d_v = hd;
    a.q_batch_stride = sq * d; a.k_batch_stride = a.v_batch_stride = sk * d;
    a.q_head_stride = a.k_head_stride = a.v_head_stride = hd;
    a.q_row_stride = a.k_row_stride = a.v_row_stride = d;
    a.o_batch_stride = sq * d; a.o_head_stride = hd; a.o_row_stride = d;
    a.causal = causal ? 1 : 0; a.kv_group = 0;
    const float scale = (float)(1.0 / std::sqrt((double)hd));
    return finish_op(fth_dev_sdpa_forward_f32(&a, scale, q->data, k->data, v->data, t->data, nullptr), t, out);
}

// ---- encoder -----------------------------------------------------------------------------------
int32_t fth_encoder_new(int64_t d_model, int64_t n_heads, int64_t d_ff, float ln_eps, int32_t causal,
                        const fth_layer_weights *layers, int64_t n_layers, fth_encoder **out) {
    FTH_ARG(out != nullptr, "encoder_new: out is NULL");
    *out = nullptr;
    if (int32_t rc = check_dims(d_model, n_heads, d_ff, n_layers)) return rc;
    FTH_ARG(n_layers == 0 || layers != nullptr, "encoder_new: layers is NULL");
    FTH_REQUIRE_DEVICE();
    fth_encoder *e = new (std::nothrow) fth_encoder();
    if (!e) return fth::set_error(FTH_ERR_KERNEL, "encoder_new: host allocation failed");
    e->stack.d_model = d_model; e->stack.n_heads = n_heads; e->stack.d_ff = d_ff;
    e->stack.eps = ln_eps; e->stack.causal = causal ? 1 : 0;
    for (int64_t i = 0; i < n_layers; ++i) {
        if (int32_t rc = e->stack.add_layer(layers[i])) {
            delete e;
            return rc;
        }
    }
    *out = e;
    return FTH_OK;
}

int32_t fth_encoder_free(fth_encoder *e) {
    if (!e) return FTH_OK;
    if (fth::available()) (void)hipDeviceSynchronize();
    for (auto &kv : e->graphs) (void)hipGraphExecDestroy(kv.second);
    for (hipGraph_t g : e->graph_templates) (void)hipGraphDestroy(g);
    delete e;
    return FTH_OK;
}

int32_t fth_encoder_forward_dev(fth_encoder *e, const float *x_dev, int64_t batch, int64_t seq, float *out_dev, fth_stream s) {
    FTH_ARG(e != nullptr, "encoder_forward: encoder is NULL");
    FTH_ARG(batch >= 0 && seq >= 0, "encoder_forward: negative extent");
    if (batch == 0 || seq == 0) return FTH_OK;
    FTH_ARG(x_dev && out_dev, "encoder_forward: NULL operand");
    FTH_ARG(x_dev != out_dev, "encoder_forward: input and output must not alias");
    std::lock_guard<std::mutex> lock(e->stack.mu);
    return e->stack.run(x_dev, batch, seq, out_dev, nullptr, s);
}

int32_t fth_encoder_forward(fth_encoder *e, const float *input, int64_t batch, int64_t seq, float *out, size_t out_cap) {
    FTH_ARG(e != nullptr, "encoder_forward: encoder is NULL");
    FTH_ARG(batch >= 0 && seq >= 0, "encoder_forward: negative extent");
    const size_t n = (size_t)batch * (size_t)seq * (size_t)e->stack.d_model;
    if (out_cap < n || (n && !out)) return fth::set_error(FTH_ERR_OUTPUT_TOO_SMALL, "encoder_forward: output buffer too small");
    if (n == 0) return FTH_OK;
    FTH_ARG(input != nullptr, "encoder_forward: input is NULL");
    FTH_REQUIRE_DEVICE();
    fth::Scratch sc;
    void *dx, *dy;
    if (int32_t rc = sc.get(&dx, n * sizeof(float))) return rc;
    if (int32_t rc = sc.get(&dy, n * sizeof(float))) return rc;
    hipStream_t st = fth::resolve_stream(nullptr);
    FTH_HIP(hipMemcpyAsync(dx, input, n * sizeof(float), hipMemcpyHostToDevice, st));
    if (int32_t rc = fth_encoder_forward_dev(e, static_cast<float *>(dx), batch, seq, static_cast<float *>(dy), nullptr)) return rc;
    FTH_HIP(hipMemcpyAsync(out, dy, n * sizeof(float), hipMemcpyDeviceToHost, st));
    return fth_stream_synchronize(nullptr);
}

int32_t fth_encoder_forward_graph(fth_encoder *e, const float *x_dev, int64_t batch, int64_t seq, float *out_dev, fth_stream s) {
    FTH_ARG(e != nullptr, "encoder_forward_graph: encoder is NULL");
    FTH_ARG(batch > 0 && seq > 0 && x_dev && out_dev && x_dev != out_dev, "encoder_forward_graph: bad arguments");
    // A run of this entry point under a rocprofiler tool library (rocprofv3 --kernel-trace) once
    // ended in a host segmentation fault inside the HIP runtime, below this function, between the
    // capture and the first replay; the same binary replays graphs without that tool. No cause
    // was found on this side of the runtime, so the combination is refused rather than retried.
    // (Checked before the device is touched, so the refusal can be tested without one.)
    if (profiler_tool_loaded())
        return fth::set_error(FTH_ERR_UNAVAILABLE, "encoder_forward_graph: HIP-graph replay is refused while a rocprofiler tool "
                                                   "library is loaded; use fth_encoder_forward_dev");
    FTH_REQUIRE_DEVICE();
    hipStream_t st = fth::resolve_stream(s);
    GraphKey key{x_dev, out_dev, batch, seq, s};
    hipGraphExec_t exec = nullptr;
    {
        std::lock_guard<std::mutex> lock(e->stack.mu);
        auto it = e->graphs.find(key);
        if (it != e->graphs.end()) exec = it->second;
    }
    if (!exec) {
        // One eager pass first: it sizes the workspaces and sets kernel attributes, neither of
        // which may happen while the stream is capturing. The capture itself records kernel
        // launches only (no memset nodes). The addresses recorded are the caller's two buffers,
        // this encoder's own activations (owned until fth_encoder_free) and the stream's GEMM
        // split-tile workspace, which is never released.
        if (int32_t rc = fth_encoder_forward_dev(e, x_dev, batch, seq, out_dev, s)) return rc;
        FTH_HIP(hipStreamSynchronize(st));
        std::lock_guard<std::mutex> lock(e->stack.mu);
        auto it = e->graphs.find(key);  // another thread may have captured the same key meanwhile
        if (it != e->graphs.end()) {
            exec = it->second;
        } else {
            FTH_HIP(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
            int32_t rc = e->stack.run(x_dev, batch, seq, out_dev, nullptr, s);
            hipGraph_t graph = nullptr;
            hipError_t ce = hipStreamEndCapture(st, &graph);
            if (rc) {
                if (graph) (void)hipGraphDestroy(graph);
                return rc;
            }
            if (ce != hipSuccess) return fth::hip_fail(ce, "hipStreamEndCapture");
            hipError_t ie = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
            if (ie != hipSuccess) {
                (void)hipGraphDestroy(graph);
                return fth::hip_fail(ie, "hipGraphInstantiate");
            }
            e->graphs[key] = exec;
            e->graph_templates.push_back(graph);  // kept until fth_encoder_free, with its executable
        }
    }
    FTH_HIP(hipGraphLaunch(exec, st));
    return FTH_OK;
}

int32_t fth_encoder_set_activation(fth_encoder *e, int32_t activation) {
    FTH_ARG(e != nullptr, "encoder_set_activation: encoder is NULL");
    FTH_ARG(activation == FTH_ACT_GELU_ERF || activation == FTH_ACT_GELU_TANH, "encoder_set_activation: unknown activation %d", activation);
    std::lock_guard<std::mutex> lock(e->stack.mu);
    FTH_ARG(e->graphs.empty(), "encoder_set_activation: a captured graph already holds the old activation");
    e->stack.gelu_epilogue = activation == FTH_ACT_GELU_TANH ? FTH_EPI_GELU_TANH : FTH_EPI_GELU;
    return FTH_OK;
}

// ---- GPT-2-shaped decoder --------------------------------------------------------------------
int32_t fth_gpt2_new(int64_t vocab, int64_t max_pos, int64_t d_model, int64_t n_heads, int64_t d_ff, float ln_eps,
                     const float *wte, const float *wpe, const fth_layer_weights *layers, int64_t n_layers,
                     const float *lnf_w, const float *lnf_b, fth_gpt2 **out) {
    FTH_ARG(out != nullptr, "gpt2_new: out is NULL");
    *out = nullptr;
    if (int32_t rc = check_dims(d_model, n_heads, d_ff, n_layers)) return rc;
    FTH_ARG(vocab > 0 && max_pos > 0 && wte && wpe, "gpt2_new: embeddings missing");
    FTH_ARG(n_layers == 0 || layers != nullptr, "gpt2_new: layers is NULL");
    FTH_REQUIRE_DEVICE();
    fth_gpt2 *g = new (std::nothrow) fth_gpt2();
    if (!g) return fth::set_error(FTH_ERR_KERNEL, "gpt2_new: host allocation failed");
    Stack &st = g->stack;
    st.d_model = d_model; st.n_heads = n_heads; st.d_ff = d_ff; st.eps = ln_eps; st.causal = 1;
    g->vocab = vocab; g->max_pos = max_pos;
    int32_t rc = st.upload(wte, vocab * d_model, &g->wte);
    if (!rc) rc = st.upload(wpe, max_pos * d_model, &g->wpe);
    if (!rc) rc = lnf_w ? st.upload(lnf_w, d_model, &g->lnf_w) : st.fill(1.f, d_model, &g->lnf_w);
    if (!rc) rc = lnf_b ? st.upload(lnf_b, d_model, &g->lnf_b) : st.fill(0.f, d_model, &g->lnf_b);
    for (int64_t i = 0; !rc && i < n_layers; ++i) rc = st.add_layer(layers[i]);
    if (!rc) {
        void *p = nullptr;
        rc = fth::pool_alloc(&p, sizeof(int64_t));
        if (!rc) {
            st.owned.push_back(p);
            g->bad = static_cast<int64_t *>(p);
        }
    }
    if (rc) {
        delete g;
        return rc;
    }
    *out = g;
    return FTH_OK;
}

// ---- GPT-2 from a safetensors checkpoint -------------------------------------------------------
namespace {

struct CheckpointReader {
    const fth_safetensors *f;
    Stack &st;
    std::string prefix;

    bool has(const std::string &name) const {
        fth_safetensors_tensor info;
        const std::string full = prefix + name;
        for (int64_t i = 0, n = fth_safetensors_count(f); i < n; ++i)
            if (full == fth_safetensors_name(f, i)) return fth_safetensors_info(f, full.c_str(), &info) == FTH_OK;
        return false;
    }
    int32_t shape(const std::string &name, int ndim, uint64_t *dims) const {
        fth_safetensors_tensor info;
        const std::string full = prefix + name;
        if (!has(name)) return fth::set_error(FTH_ERR_CORRUPT, "checkpoint has no tensor '%s'", full.c_str());
        if (int32_t rc = fth_safetensors_info(f, full.c_str(), &info)) return rc;
        if (info.ndim != ndim) return fth::set_error(FTH_ERR_CORRUPT, "checkpoint tensor '%s' has %d dimensions, expected %d", full.c_str(), info.ndim, ndim);
        for (int i = 0; i < ndim; ++i) dims[i] = info.shape[i];
        return FTH_OK;
    }
    // Reads `name` (shape [d0] or [d0, d1] as stored) into a new device block owned by the stack.
    int32_t load(const std::string &name, uint64_t d0, uint64_t d1, bool transpose, float **dev) {
        uint64_t dims[2] = {0, 0};
        const int ndim = d1 ? 2 : 1;
        if (int32_t rc = shape(name, ndim, dims)) return rc;
        if (dims[0] != d0 || (ndim == 2 && dims[1] != d1))
            return fth::set_error(FTH_ERR_CORRUPT, "checkpoint tensor '%s%s' is [%llu, %llu], expected [%llu, %llu]", prefix.c_str(), name.c_str(),
                                  (unsigned long long)dims[0], (unsigned long long)dims[1], (unsigned long long)d0, (unsigned long long)d1);
        const size_t n = (size_t)(d0 * (d1 ? d1 : 1));
        void *p = nullptr;
        if (int32_t rc = fth::pool_alloc(&p, n * sizeof(float))) return rc;
        st.owned.push_back(p);
        *dev = static_cast<float *>(p);
        return fth_safetensors_read_f32_dev(f, (prefix + name).c_str(), transpose ? 1 : 0, *dev, n, nullptr);
    }
};

}  // namespace

int32_t fth_gpt2_from_safetensors(const fth_safetensors *f, int64_t n_heads, float ln_eps, int32_t activation, fth_gpt2 **out) {
    FTH_ARG(out != nullptr, "gpt2_from_safetensors: out is NULL");
    *out = nullptr;
    FTH_ARG(f != nullptr, "gpt2_from_safetensors: file is NULL");
    FTH_ARG(activation == FTH_ACT_GELU_ERF || activation == FTH_ACT_GELU_TANH, "gpt2_from_safetensors: unknown activation %d", activation);
    FTH_REQUIRE_DEVICE();
    fth_gpt2 *g = new (std::nothrow) fth_gpt2();
    if (!g) return fth::set_error(FTH_ERR_KERNEL, "gpt2_from_safetensors: host allocation failed");
    Stack &st = g->stack;
    CheckpointReader rd{f, st, ""};
    if (!rd.has("wte.weight")) rd.prefix = "transformer.";
    uint64_t e[2], pdim[2], fc[2];
    int32_t rc = rd.shape("wte.weight", 2, e);
    if (!rc) rc = rd.shape("wpe.weight", 2, pdim);
    int64_t n_layers = 0;
    while (!rc && rd.has("h." + std::to_string(n_layers) + ".ln_1.weight")) ++n_layers;
    const uint64_t d = e[1];
    uint64_t d_ff = d;
    if (!rc && n_layers > 0) {
        rc = rd.shape("h.0.mlp.c_fc.weight", 2, fc);
        d_ff = fc[1];
    }
    if (!rc && pdim[1] != d) rc = fth::set_error(FTH_ERR_CORRUPT, "checkpoint: wpe.weight width %llu differs from wte.weight width %llu",
                                                 (unsigned long long)pdim[1], (unsigned long long)d);
    if (!rc) rc = check_dims((int64_t)d, n_heads, (int64_t)d_ff, n_layers);
    if (!rc) {
        st.d_model = (int64_t)d; st.n_heads = n_heads; st.d_ff = (int64_t)d_ff; st.eps = ln_eps; st.causal = 1;
        st.gelu_epilogue = activation == FTH_ACT_GELU_TANH ? FTH_EPI_GELU_TANH : FTH_EPI_GELU;
        g->vocab = (int64_t)e[0]; g->max_pos = (int64_t)pdim[0];
        rc = rd.load("wte.weight", e[0], d, false, &g->wte);
    }
    if (!rc) rc = rd.load("wpe.weight", pdim[0], d, false, &g->wpe);
    if (!rc) rc = rd.load("ln_f.weight", d, 0, false, &g->lnf_w);
    if (!rc) rc = rd.load("ln_f.bias", d, 0, false, &g->lnf_b);
    for (int64_t i = 0; !rc && i < n_layers; ++i) {
        const std::string h = "h." + std::to_string(i) + ".";
        LayerDev L = {};
        // Conv1D weights are stored [in, out]; the linear kernels read [out, in], so c_attn.weight^T is the packed
        // [3d, d] query / key / value matrix as it stands.
        rc = rd.load(h + "ln_1.weight", d, 0, false, &L.ln1_w);
        if (!rc) rc = rd.load(h + "ln_1.bias", d, 0, false, &L.ln1_b);
        if (!rc) rc = rd.load(h + "attn.c_attn.weight", d, 3 * d, true, &L.wqkv);
        if (!rc) rc = rd.load(h + "attn.c_attn.bias", 3 * d, 0, false, &L.bqkv);
        if (!rc) rc = rd.load(h + "attn.c_proj.weight", d, d, true, &L.wo);
        if (!rc) rc = rd.load(h + "attn.c_proj.bias", d, 0, false, &L.bo);
        if (!rc) rc = rd.load(h + "ln_2.weight", d, 0, false, &L.ln2_w);
        if (!rc) rc = rd.load(h + "ln_2.bias", d, 0, false, &L.ln2_b);
        if (!rc) rc = rd.load(h + "mlp.c_fc.weight", d, d_ff, true, &L.w1);
        if (!rc) rc = rd.load(h + "mlp.c_fc.bias", d_ff, 0, false, &L.b1);
        if (!rc) rc = rd.load(h + "mlp.c_proj.weight", d_ff, d, true, &L.w2);
        if (!rc) rc = rd.load(h + "mlp.c_proj.bias", d, 0, false, &L.b2);
        if (!rc) st.layers.push_back(L);
    }
    if (!rc) {
        void *p = nullptr;
        rc = fth::pool_alloc(&p, sizeof(int64_t));
        if (!rc) {
            st.owned.push_back(p);
            g->bad = static_cast<int64_t *>(p);
        }
    }
    if (rc) {
        delete g;
        return rc;
    }
    *out = g;
    return FTH_OK;
}

int32_t fth_gpt2_from_statedict(const fth_statedict *f, int64_t n_heads, float ln_eps, int32_t activation, fth_gpt2 **out) {
    // The two containers share their handle type: the reader only asks for names, shapes and device reads.
    return fth_gpt2_from_safetensors(f, n_heads, ln_eps, activation, out);
}

int32_t fth_gpt2_dims(const fth_gpt2 *g, int64_t *vocab, int64_t *max_pos, int64_t *d_model, int64_t *n_heads, int64_t *d_ff,
                      int64_t *n_layers) {
    FTH_ARG(g != nullptr, "gpt2_dims: model is NULL");
    if (vocab) *vocab = g->vocab;
    if (max_pos) *max_pos = g->max_pos;
    if (d_model) *d_model = g->stack.d_model;
    if (n_heads) *n_heads = g->stack.n_heads;
    if (d_ff) *d_ff = g->stack.d_ff;
    if (n_layers) *n_layers = (int64_t)g->stack.layers.size();
    return FTH_OK;
}

int32_t fth_gpt2_set_activation(fth_gpt2 *g, int32_t activation) {
    FTH_ARG(g != nullptr, "gpt2_set_activation: model is NULL");
    FTH_ARG(activation == FTH_ACT_GELU_ERF || activation == FTH_ACT_GELU_TANH, "gpt2_set_activation: unknown activation %d", activation);
    std::lock_guard<std::mutex> lock(g->stack.mu);
    g->stack.gelu_epilogue = activation == FTH_ACT_GELU_TANH ? FTH_EPI_GELU_TANH : FTH_EPI_GELU;
    return FTH_OK;
}

int32_t fth_gpt2_free(fth_gpt2 *g) {
    if (!g) return FTH_OK;
    if (fth::available()) (void)hipDeviceSynchronize();
    delete g;
    return FTH_OK;
}

int32_t fth_gpt2_forward_dev(fth_gpt2 *g, const double *ids_dev, int64_t batch, int64_t seq, float *logits_dev,
                             float *argmax_dev, fth_stream s) {
    FTH_ARG(g != nullptr, "gpt2_forward: model is NULL");
    FTH_ARG(batch >= 0 && seq >= 0, "gpt2_forward: negative extent");
    if (batch == 0 || seq == 0) return FTH_OK;
    FTH_ARG(ids_dev != nullptr, "gpt2_forward: ids is NULL");
    FTH_ARG(seq <= g->max_pos, "gpt2_forward: seq %lld exceeds the %lld learned positions", (long long)seq, (long long)g->max_pos);
    Stack &st = g->stack;
    std::lock_guard<std::mutex> lock(st.mu);
    const int64_t T = batch * seq, d = st.d_model;
    if (T > g->tokens_cap) {
        void *p0 = nullptr, *p1 = nullptr;
        if (int32_t rc = fth::pool_alloc(&p0, (size_t)T * d * sizeof(float))) return rc;
        st.owned.push_back(p0);
        if (int32_t rc = fth::pool_alloc(&p1, (size_t)T * d * sizeof(float))) return rc;
        st.owned.push_back(p1);
        g->x0 = static_cast<float *>(p0);
        g->hidden = static_cast<float *>(p1);
        g->tokens_cap = T;
    }
    float *logits = logits_dev;
    if (!logits && argmax_dev) {
        if (T > g->logits_cap) {
            void *p = nullptr;
            if (int32_t rc = fth::pool_alloc(&p, (size_t)T * (size_t)g->vocab * sizeof(float))) return rc;
            st.owned.push_back(p);
            g->logits = static_cast<float *>(p);
            g->logits_cap = T;
        }
        logits = g->logits;
    }
    if (argmax_dev && T > g->group_max_cap) {  // row maxima per column group of the logits, for the fused argmax
        void *p = nullptr;
        if (int32_t rc = fth::pool_alloc(&p, (size_t)fth_dev_linear_argmax_workspace_floats(T, g->vocab) * sizeof(float))) return rc;
        st.owned.push_back(p);
        g->group_max = static_cast<float *>(p);
        g->group_max_cap = T;
    }
    int32_t rc;
    if ((rc = fth_dev_embedding_add_f32(g->wte, g->vocab, g->wpe, g->max_pos, ids_dev, T, seq, d, g->x0, g->bad, s))) return rc;
    const float *x = nullptr;
    if ((rc = st.run(g->x0, batch, seq, nullptr, &x, s))) return rc;
    if ((rc = fth_dev_layer_norm_f32(x, g->lnf_w, g->lnf_b, g->hidden, T, d, st.eps, s))) return rc;
    if (logits) {
        // Tied head: the [vocab, d_model] embedding table is exactly the [out, in] weight layout.
        if (argmax_dev) {
            if ((rc = fth_dev_linear_argmax_f32(g->hidden, g->wte, T, g->vocab, d, logits, argmax_dev, g->group_max,
                                                fth_dev_linear_argmax_workspace_floats(g->group_max_cap, g->vocab), s)))
                return rc;
        } else {
            fth_gemm_desc gd = linear_desc(T, g->vocab, d, FTH_EPI_NONE);
            if ((rc = fth_dev_gemm_f32(&gd, 1.f, g->hidden, g->wte, logits, nullptr, nullptr, s))) return rc;
        }
    }
    return FTH_OK;
}

const float *fth_gpt2_hidden_dev(const fth_gpt2 *g) { return g ? g->hidden : nullptr; }

int32_t fth_gpt2_bad_index(const fth_gpt2 *g, int64_t *position) {
    FTH_ARG(g != nullptr && position != nullptr, "gpt2_bad_index: NULL argument");
    FTH_REQUIRE_DEVICE();
    FTH_HIP(hipMemcpy(position, g->bad, sizeof(int64_t), hipMemcpyDeviceToHost));
    return FTH_OK;
}

}  // extern "C"
