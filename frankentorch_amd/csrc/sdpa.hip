// Fused scaled-dot-product attention forward for gfx950 (fp32 on v_mfma_f32_32x32x2_f32).
//
// replaces sdpa_forward_f32 / sdpa_forward_f64 (crates/ft-kernel-cpu/src/lib.rs:5200-5284,
// 4572-4651): scores = Q.K^T, scale AFTER the product, row softmax over the first
// limit = min(qi + 1, seq_k) keys when causal (all seq_k otherwise), entries past the limit are
// exactly zero, out = P.V. The reference materialises a [64, seq_k] score tile per block and
// normalises P before the second product; this kernel never materialises scores: it walks the
// keys in tiles of 32 with an online softmax (running max m, running sum l, rescaled
// accumulator) and divides by l once at the end. Same mathematics, different rounding order:
// covered by the 2e-5 tolerance of the parity tests.
//
// Layout of the MFMA work (one wavefront = 32 queries, a block = 4 wavefronts = 128 queries that
// share each K/V tile through LDS):
//   S^T[key, query] = K_tile . Q^T      A operand = K rows from LDS (one 128-bit read feeds four
//                                       MFMAs), B operand = the wavefront's Q rows, resident in
//                                       registers for the whole kernel.
//   In the 32x32 accumulator layout a lane then holds, for ONE query (lane % 32), 16 of the 32
//   keys; the other 16 sit in lane ^ 32. Row max / row sum are 16 in-lane steps plus one
//   cross-half exchange, and the per-query rescale factor is lane-local.
//   O^T[d, query] += V_tile^T . P^T     B operand = the lane's own P registers, unchanged: the
//                                       k index of MFMA step r is exactly the key that register r
//                                       holds, so P never goes through LDS. A operand = V rows
//                                       from LDS, one vector read (d = NDT * (lane % 32) + e)
//                                       feeding the NDT d-tiles.
// No atomics, no split over keys across wavefronts: bitwise repeatable.
//
// Tile order: blocks of one (batch, head) are given to one XCD so that its K/V (<= a few MB)
// stay in that XCD's L2, and the long (late) query blocks of a causal problem are issued first.

#include <type_traits>

#include "common.hpp"

namespace {

constexpr int kWave = 64;
constexpr int kXcds = 8;
constexpr int kBQ = 128;  // queries per block (4 wavefronts x 32)
constexpr int kBC = 32;   // keys per tile

using Acc16 = float __attribute__((ext_vector_type(16)));

struct SdpaArgs {
    const void *q, *k, *v;
    void *out;
    fth_sdpa_desc d;
    double scale;
    int q_blocks;
};

template <int N> struct VecN;
template <> struct VecN<1> { using type = float; };
template <> struct VecN<2> { using type = float2; };
template <> struct VecN<4> { using type = float4; };
__device__ __forceinline__ float vecn_get(const float &v, int) { return v; }
__device__ __forceinline__ float vecn_get(const float2 &v, int e) { return e == 0 ? v.x : v.y; }
__device__ __forceinline__ float vecn_get(const float4 &v, int e) { return e == 0 ? v.x : e == 1 ? v.y : e == 2 ? v.z : v.w; }
__device__ __forceinline__ float f4_get(const float4 &v, int e) { return e == 0 ? v.x : e == 1 ? v.y : e == 2 ? v.z : v.w; }

template <int D>
__global__ __launch_bounds__(256, 2) void sdpa_mfma_kernel(const SdpaArgs p) {
    constexpr int NDT = D / 32;        // 32-wide d-tiles of the output
    constexpr int KP = D + 4;          // K tile row pitch (odd number of 16-byte vectors)
    constexpr int VP = D + 8;          // V tile row pitch (rows j and j+4 land 32 banks apart)
    constexpr int KT = kBC * KP;       // floats per K tile
    constexpr int VT = kBC * VP;
    constexpr int NV = kBC * (D / 4) / 256;  // float4 per thread per tile
    static_assert(kBC * (D / 4) % 256 == 0, "tile must divide over the block");
    using VV = typename VecN<NDT>::type;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    float *Ks = reinterpret_cast<float *>(smem_raw);  // [2][kBC][KP]
    float *Vs = Ks + 2 * KT;                          // [2][kBC][VP]

    const fth_sdpa_desc &d = p.d;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lq = lane & 31, half = lane >> 5;

    // ---- which (bh, query block) ----
    int64_t bh;
    int qb;
    {
        const int64_t pid = blockIdx.x;
        if (d.num_bh % kXcds == 0) {
            const int64_t xcd = pid % kXcds, w = pid / kXcds;
            bh = (w / p.q_blocks) * kXcds + xcd;
            qb = (int)(w % p.q_blocks);
        } else {
            bh = pid / p.q_blocks;
            qb = (int)(pid % p.q_blocks);
        }
        qb = p.q_blocks - 1 - qb;  // longest causal rows first
    }
    const int64_t b = bh / d.heads, h = bh % d.heads;
    const float *Q = static_cast<const float *>(p.q) + b * d.q_batch_stride + h * d.q_head_stride;
    const float *K = static_cast<const float *>(p.k) + b * d.k_batch_stride + h * d.k_head_stride;
    const float *Vg = static_cast<const float *>(p.v) + b * d.v_batch_stride + h * d.v_head_stride;
    float *O = static_cast<float *>(p.out) + b * d.o_batch_stride + h * d.o_head_stride;
    const float scale = (float)p.scale;

    const int64_t q_blk0 = (int64_t)qb * kBQ;
    const int64_t q_wave0 = q_blk0 + wave * 32;
    const int64_t qi = q_wave0 + lq;  // this lane's query
    const bool q_live = qi < d.seq_q;

    // ---- Q rows into registers: lane holds Q[qi][8t + 4*half + e] ----
    float4 qr[D / 8];
#pragma unroll
    for (int t = 0; t < D / 8; ++t) {
        qr[t] = q_live ? *reinterpret_cast<const float4 *>(Q + qi * d.q_row_stride + 8 * t + 4 * half)
                       : make_float4(0.f, 0.f, 0.f, 0.f);
    }

    // ---- key range ----
    int64_t blk_last_q = q_blk0 + kBQ - 1;
    if (blk_last_q > d.seq_q - 1) blk_last_q = d.seq_q - 1;
    int64_t k_end = d.seq_k;  // exclusive
    if (d.causal && blk_last_q + 1 < k_end) k_end = blk_last_q + 1;
    const int num_kt = (int)((k_end + kBC - 1) / kBC);
    int64_t wave_last_q = q_wave0 + 31;
    if (wave_last_q > d.seq_q - 1) wave_last_q = d.seq_q - 1;

    float4 kst[NV], vst[NV];
    auto load_tile = [&](int kt) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int vid = tid + i * 256;
            const int row = vid / (D / 4), c = vid % (D / 4);
            const int64_t key = (int64_t)kt * kBC + row;
            if (key < d.seq_k) {
                kst[i] = *reinterpret_cast<const float4 *>(K + key * d.k_row_stride + 4 * c);
                vst[i] = *reinterpret_cast<const float4 *>(Vg + key * d.v_row_stride + 4 * c);
            } else {
                kst[i] = make_float4(0.f, 0.f, 0.f, 0.f);
                vst[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int vid = tid + i * 256;
            const int row = vid / (D / 4), c = vid % (D / 4);
            *reinterpret_cast<float4 *>(Ks + buf * KT + row * KP + 4 * c) = kst[i];
            *reinterpret_cast<float4 *>(Vs + buf * VT + row * VP + 4 * c) = vst[i];
        }
    };

    Acc16 o[NDT];
#pragma unroll
    for (int e = 0; e < NDT; ++e)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[e][r] = 0.f;
    float m_run = -__builtin_inff();
    float l_run = 0.f;

    if (num_kt > 0) {
        load_tile(0);
        store_tile(0);
    }
    __syncthreads();

    for (int kt = 0; kt < num_kt; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < num_kt) load_tile(kt + 1);
        const int64_t key0 = (int64_t)kt * kBC;
        // A wavefront whose every query precedes this tile's first key has nothing to add.
        const bool wave_active = !d.causal || key0 <= wave_last_q;
        if (wave_active) {
            // ---- S^T = K_tile . Q^T ----
            Acc16 s;
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] = 0.f;
            const float *kp = Ks + buf * KT + lq * KP + 4 * half;
#pragma unroll
            for (int t = 0; t < D / 8; ++t) {
                const float4 kv = *reinterpret_cast<const float4 *>(kp + 8 * t);
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.x, qr[t].x, s, 0, 0, 0);
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.y, qr[t].y, s, 0, 0, 0);
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.z, qr[t].z, s, 0, 0, 0);
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.w, qr[t].w, s, 0, 0, 0);
            }
            // ---- scale, mask, online softmax (lane-local query) ----
            const bool need_mask = (d.causal && key0 + kBC - 1 > q_wave0) || (key0 + kBC > d.seq_k);
            float sv[16];
            float mt = -__builtin_inff();
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float x = s[r] * scale;
                if (need_mask) {
                    const int64_t key = key0 + 8 * (r >> 2) + 4 * half + (r & 3);
                    if ((d.causal && key > qi) || key >= d.seq_k) x = -__builtin_inff();
                }
                sv[r] = x;
                mt = fmaxf(mt, x);
            }
            mt = fmaxf(mt, __shfl_xor(mt, 32, kWave));
            const float m_new = fmaxf(m_run, mt);
            const float alpha = expf(m_run - m_new);
            float psum = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float e = expf(sv[r] - m_new);
                sv[r] = e;
                psum += e;
            }
            psum += __shfl_xor(psum, 32, kWave);
            l_run = l_run * alpha + psum;
            m_run = m_new;
            if (__any(alpha != 1.0f)) {
#pragma unroll
                for (int e = 0; e < NDT; ++e)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o[e][r] *= alpha;
            }
            // ---- O^T += V_tile^T . P^T ----
            const float *vp = Vs + buf * VT + (4 * half) * VP + NDT * lq;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const VV vv = *reinterpret_cast<const VV *>(vp + (8 * (r >> 2) + (r & 3)) * VP);
#pragma unroll
                for (int e = 0; e < NDT; ++e)
                    o[e] = __builtin_amdgcn_mfma_f32_32x32x2f32(vecn_get(vv, e), sv[r], o[e], 0, 0, 0);
            }
        }
        if (kt + 1 < num_kt) store_tile(buf ^ 1);
        __syncthreads();
    }

    // ---- normalise and store: lane owns query qi, d = NDT * rho + e ----
    if (q_live) {
        float *orow = O + qi * d.o_row_stride;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int rho = 8 * (r >> 2) + 4 * half + (r & 3);
            float ov[NDT];
#pragma unroll
            for (int e = 0; e < NDT; ++e) ov[e] = (num_kt > 0) ? o[e][r] / l_run : 0.f;
            if constexpr (NDT == 4) *reinterpret_cast<float4 *>(orow + 4 * rho) = make_float4(ov[0], ov[1], ov[2], ov[3]);
            else if constexpr (NDT == 2) *reinterpret_cast<float2 *>(orow + 2 * rho) = make_float2(ov[0], ov[1]);
            else orow[rho] = ov[0];
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Generic variant: any d_k / d_v / strides, float or double. One wavefront per query row; keys
// in chunks of 64 (lane j scores key j); the same online softmax. Used for fp64 and for head
// sizes the MFMA variant does not cover.
// ---------------------------------------------------------------------------------------------
template <typename T> __device__ __forceinline__ T t_exp(T x);
template <> __device__ __forceinline__ float t_exp<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ double t_exp<double>(double x) { return exp(x); }
template <typename T> __device__ __forceinline__ T t_max(T a, T b);
template <> __device__ __forceinline__ float t_max<float>(float a, float b) { return fmaxf(a, b); }
template <> __device__ __forceinline__ double t_max<double>(double a, double b) { return fmax(a, b); }

template <typename T, int MAXDV_PER_LANE>
__global__ __launch_bounds__(64) void sdpa_generic_kernel(const SdpaArgs p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T *qs = reinterpret_cast<T *>(smem_raw);  // [d_k]
    const fth_sdpa_desc &d = p.d;
    const int lane = threadIdx.x;
    const int64_t row = blockIdx.x;
    const int64_t bh = row / d.seq_q, qi = row % d.seq_q;
    const int64_t b = bh / d.heads, h = bh % d.heads;
    const T *Q = static_cast<const T *>(p.q) + b * d.q_batch_stride + h * d.q_head_stride + qi * d.q_row_stride;
    const T *K = static_cast<const T *>(p.k) + b * d.k_batch_stride + h * d.k_head_stride;
    const T *V = static_cast<const T *>(p.v) + b * d.v_batch_stride + h * d.v_head_stride;
    T *O = static_cast<T *>(p.out) + b * d.o_batch_stride + h * d.o_head_stride + qi * d.o_row_stride;
    const T scale = (T)p.scale;
    for (int64_t c = lane; c < d.d_k; c += 64) qs[c] = Q[c];
    __syncthreads();
    int64_t limit = d.seq_k;
    if (d.causal && qi + 1 < limit) limit = qi + 1;
    T acc[MAXDV_PER_LANE];
#pragma unroll
    for (int i = 0; i < MAXDV_PER_LANE; ++i) acc[i] = T(0);
    const T ninf = (T)-__builtin_inf();
    T m_run = ninf, l_run = T(0);
    for (int64_t k0 = 0; k0 < limit; k0 += 64) {
        const int64_t key = k0 + lane;
        T sc = ninf;
        if (key < limit) {
            const T *kr = K + key * d.k_row_stride;
            T dot = T(0);
            for (int64_t c = 0; c < d.d_k; ++c) dot += qs[c] * kr[c];
            sc = dot * scale;
        }
        T mt = sc;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) mt = t_max(mt, __shfl_xor(mt, off, 64));
        const T m_new = t_max(m_run, mt);
        const T alpha = t_exp(m_run - m_new);
        const T pj = (key < limit) ? t_exp(sc - m_new) : T(0);
        T ps = pj;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) ps += __shfl_xor(ps, off, 64);
        l_run = l_run * alpha + ps;
        m_run = m_new;
#pragma unroll
        for (int i = 0; i < MAXDV_PER_LANE; ++i) acc[i] *= alpha;
        const int64_t nk = (limit - k0) < 64 ? (limit - k0) : 64;
        for (int64_t j = 0; j < nk; ++j) {
            const T pv = __shfl(pj, (int)j, 64);
            const T *vr = V + (k0 + j) * d.v_row_stride;
#pragma unroll
            for (int i = 0; i < MAXDV_PER_LANE; ++i) {
                const int64_t c = lane + (int64_t)i * 64;
                if (c < d.d_v) acc[i] += pv * vr[c];
            }
        }
    }
#pragma unroll
    for (int i = 0; i < MAXDV_PER_LANE; ++i) {
        const int64_t c = lane + (int64_t)i * 64;
        if (c < d.d_v) O[c] = (limit > 0) ? acc[i] / l_run : T(0);
    }
}

template <int D> int32_t launch_mfma(const SdpaArgs &a, hipStream_t st) {
    constexpr size_t smem = (size_t)2 * kBC * ((D + 4) + (D + 8)) * sizeof(float);
    auto kern = sdpa_mfma_kernel<D>;
    static bool attr_set = false;
    if (!attr_set) {
        FTH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    const int64_t grid = a.d.num_bh * a.q_blocks;
    FTH_ARG(grid <= 2147483647LL, "sdpa: grid too large");
    kern<<<dim3((unsigned)grid), dim3(256), smem, st>>>(a);
    FTH_CHECK_LAUNCH("sdpa_mfma");
    return FTH_OK;
}

template <typename T>
int32_t sdpa_entry(const fth_sdpa_desc *d, double scale, const T *q, const T *k, const T *v, T *out, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(d != nullptr, "sdpa: desc is NULL");
    FTH_ARG(d->num_bh >= 0 && d->seq_q >= 0 && d->seq_k >= 0 && d->d_k >= 0 && d->d_v >= 0, "sdpa: negative extent");
    FTH_ARG(d->heads >= 1 && d->num_bh % d->heads == 0, "sdpa: heads (%lld) must divide num_bh (%lld)",
            (long long)d->heads, (long long)d->num_bh);
    if (d->num_bh == 0 || d->seq_q == 0 || d->d_v == 0) return FTH_OK;
    FTH_ARG(q && k && v && out, "sdpa: NULL operand");
    hipStream_t st = fth::resolve_stream(s);
    SdpaArgs a;
    a.q = q; a.k = k; a.v = v; a.out = out; a.d = *d; a.scale = scale;
    a.q_blocks = (int)fth::ceil_div(d->seq_q, kBQ);
    auto al16 = [](const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; };
    auto m4 = [](int64_t x) { return x % 4 == 0; };
    if constexpr (std::is_same<T, float>::value) {
        const bool strides_ok = m4(d->q_batch_stride) && m4(d->q_head_stride) && m4(d->q_row_stride) &&
                                m4(d->k_batch_stride) && m4(d->k_head_stride) && m4(d->k_row_stride) &&
                                m4(d->v_batch_stride) && m4(d->v_head_stride) && m4(d->v_row_stride) &&
                                m4(d->o_batch_stride) && m4(d->o_head_stride) && m4(d->o_row_stride) &&
                                al16(q) && al16(k) && al16(v) && al16(out);
        if (strides_ok && d->d_k == d->d_v && d->seq_k > 0) {
            if (d->d_k == 128) return launch_mfma<128>(a, st);
            if (d->d_k == 64) return launch_mfma<64>(a, st);
            if (d->d_k == 32) return launch_mfma<32>(a, st);
        }
    }
    FTH_ARG(d->d_v <= 64 * 8, "sdpa: d_v %lld exceeds the generic kernel's limit of 512", (long long)d->d_v);
    const int64_t rows = d->num_bh * d->seq_q;
    FTH_ARG(rows <= 2147483647LL, "sdpa: grid too large");
    const size_t smem = (size_t)(d->d_k > 0 ? d->d_k : 1) * sizeof(T);
    FTH_ARG(smem <= 64 * 1024, "sdpa: d_k %lld too large for the generic kernel", (long long)d->d_k);
    if (d->d_v <= 128) sdpa_generic_kernel<T, 2><<<dim3((unsigned)rows), dim3(64), smem, st>>>(a);
    else sdpa_generic_kernel<T, 8><<<dim3((unsigned)rows), dim3(64), smem, st>>>(a);
    FTH_CHECK_LAUNCH("sdpa_generic");
    return FTH_OK;
}

}  // namespace

extern "C" {

void fth_sdpa_desc_contiguous(fth_sdpa_desc *d, int64_t num_bh, int64_t seq_q, int64_t seq_k, int64_t d_k,
                              int64_t d_v, int32_t causal) {
    if (!d) return;
    d->num_bh = num_bh;
    d->heads = 1;
    d->seq_q = seq_q; d->seq_k = seq_k; d->d_k = d_k; d->d_v = d_v;
    d->q_batch_stride = seq_q * d_k; d->q_head_stride = 0; d->q_row_stride = d_k;
    d->k_batch_stride = seq_k * d_k; d->k_head_stride = 0; d->k_row_stride = d_k;
    d->v_batch_stride = seq_k * d_v; d->v_head_stride = 0; d->v_row_stride = d_v;
    d->o_batch_stride = seq_q * d_v; d->o_head_stride = 0; d->o_row_stride = d_v;
    d->causal = causal;
    d->reserved = 0;
}

int32_t fth_dev_sdpa_forward_f32(const fth_sdpa_desc *d, float scale, const float *q, const float *k, const float *v,
                                 float *out, fth_stream s) {
    return sdpa_entry<float>(d, (double)scale, q, k, v, out, s);
}

int32_t fth_dev_sdpa_forward_f64(const fth_sdpa_desc *d, double scale, const double *q, const double *k,
                                 const double *v, double *out, fth_stream s) {
    return sdpa_entry<double>(d, scale, q, k, v, out, s);
}

}  // extern "C"
