// Dense contraction on the gfx950 matrix cores: C = alpha * A * op(B) (+ bias, GELU, residual).
//
//   fp32: v_mfma_f32_32x32x2_f32   (32x32 output tile per wavefront instruction, k = 2)
//   fp64: v_mfma_f64_16x16x4_f64   (16x16 output tile, k = 4)
//
// Data path. A block owns a BM x BN tile of C. Both operands are staged in LDS K-CONTIGUOUS
// (As[BM][BK+pad], Bs[BN][BK+pad]), so a lane fetches its MFMA operands with one 128-bit LDS
// read: that vector holds EPV consecutive k for the lane's row, and feeds EPV successive MFMAs.
// Which k lands in which MFMA is irrelevant as long as A and B agree, and they do because both
// use the same (lane / MT, element) -> k map. The pad (one vector per row) makes the row pitch
// an odd number of vectors, which spreads the 16 rows of a read pass over all 64 banks.
// Global -> LDS goes through registers, one K-tile ahead (two LDS buffers, one barrier per
// K-tile): the loads of tile t+1 are issued before the MFMAs of tile t.
//   A, and B stored [n, k] (trans_b): 128-bit global loads along k.
//   B stored [k, n]: each thread reads EPV consecutive k of ONE column with scalar loads (the
//   wavefront covers 64 consecutive columns, so every load instruction is one 256-byte run) and
//   writes them to LDS as a single vector. No transpose pass, no bank conflicts.
// The accumulators never leave registers; K is never split, so the sum order of an output
// element depends on the shape and the tile configuration only: bitwise repeatable.
//
// Tile order. Consecutive workgroup ids land on different XCDs (8 per device, each with its own
// L2), so the id is first remapped to give each XCD one contiguous range of tiles, and within
// the range tiles are walked in groups of GROUP_M tile-rows so that concurrently resident blocks
// share A row-panels and B column-panels in that XCD's L2.
//
// replaces gemm::sgemm / dgemm / sgemm_bt / dgemm_bt (crates/ft-kernel-cpu/src/lib.rs:1310-1338,
// 107-138, 1430-1481, 201-255), the per-batch loop of bmm (:38572-38606) and the bias pass of
// linear_tensor_f32 (:17336-17351).

#include <type_traits>

#include "common.hpp"

namespace {

constexpr int kWave = 64;
constexpr int kXcds = 8;
constexpr int kGroupM = 8;

template <typename T> struct Mfma;
template <> struct Mfma<float> {
    static constexpr int MT = 32;   // output tile edge
    static constexpr int KG = 2;    // k-groups across the wavefront (64 / MT)
    static constexpr int EPV = 4;   // elements per 128-bit vector
    static constexpr int ACC = 16;  // accumulator elements per lane
    using Acc = float __attribute__((ext_vector_type(16)));
    using V = float4;
    __device__ __forceinline__ static Acc mma(float a, float b, Acc c) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
    // Row (within the 32x32 tile) of accumulator element r held by `lane`; the column is lane % 32.
    __device__ __forceinline__ static int acc_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }
    __device__ __forceinline__ static float elem(const V &v, int j) { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; }
    __device__ __forceinline__ static V zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
    __device__ __forceinline__ static V make(const float *e) { return make_float4(e[0], e[1], e[2], e[3]); }
    __device__ __forceinline__ static float gelu(float x) { return (0.5f * x) * (1.0f + erff(x * 0.70710678118654752440f)); }
};
template <> struct Mfma<double> {
    static constexpr int MT = 16;
    static constexpr int KG = 4;
    static constexpr int EPV = 2;
    static constexpr int ACC = 4;
    using Acc = double __attribute__((ext_vector_type(4)));
    using V = double2;
    __device__ __forceinline__ static Acc mma(double a, double b, Acc c) {
        return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
    }
    // 16x16 f64 tile: accumulator element r of `lane` is row 4 * r + lane / 16, column lane % 16.
    __device__ __forceinline__ static int acc_row(int r, int lane) { return 4 * r + (lane >> 4); }
    __device__ __forceinline__ static double elem(const V &v, int j) { return j == 0 ? v.x : v.y; }
    __device__ __forceinline__ static V zero() { return make_double2(0.0, 0.0); }
    __device__ __forceinline__ static V make(const double *e) { return make_double2(e[0], e[1]); }
    __device__ __forceinline__ static double gelu(double x) { return (0.5 * x) * (1.0 + erf(x * 0.70710678118654752440)); }
};

template <typename T> struct GemmArgs {
    const T *a;
    const T *b;
    T *c;
    const T *bias;
    const T *residual;
    int64_t m, n, k;
    int64_t lda, ldb, ldc;
    int64_t stride_a, stride_b, stride_c;
    T alpha;
    int tiles_m, tiles_n;
    int epilogue;
    int use_alpha;
};

// Maps the hardware workgroup id to a (tile_m, tile_n) pair: XCD-contiguous, then grouped.
__device__ __forceinline__ void tile_of_block(int pid, int tiles_m, int tiles_n, int &tm, int &tn) {
    const int nblk = tiles_m * tiles_n;
    const int per = nblk / kXcds, rem = nblk % kXcds;
    const int xcd = pid % kXcds, q = pid / kXcds;
    const int id = q + xcd * per + (xcd < rem ? xcd : rem);
    const int group = kGroupM * tiles_n;
    const int g = id / group;
    const int first_m = g * kGroupM;
    const int gm = (tiles_m - first_m) < kGroupM ? (tiles_m - first_m) : kGroupM;
    const int in_g = id - g * group;
    tm = first_m + in_g % gm;
    tn = in_g / gm;
}

template <typename T, int BM, int BN, int BK, int WM, int WN, bool TRANS_B, bool VEC>
__global__ __launch_bounds__(WM *WN *kWave) void gemm_kernel(const GemmArgs<T> p) {
    using M = Mfma<T>;
    using V = typename M::V;
    constexpr int MT = M::MT, KG = M::KG, EPV = M::EPV;
    constexpr int NT = WM * WN * kWave;
    constexpr int S = BK + EPV;          // LDS row pitch in elements (odd number of vectors)
    constexpr int KV = BK / EPV;         // vectors per tile row
    constexpr int KCH = KG * EPV;        // k covered by one operand vector fetch
    constexpr int WTM = BM / WM, WTN = BN / WN;
    constexpr int TM = WTM / MT, TN = WTN / MT;
    static_assert(BK % KCH == 0, "BK must be a multiple of the per-fetch k extent");
    static_assert((KV & 1) == 0, "BK / EPV must be even so the padded pitch is an odd vector count");
    static_assert(WTM % MT == 0 && WTN % MT == 0, "wave tile must be a whole number of MFMA tiles");
    constexpr int A_VECS = BM * KV / NT;  // vectors of A each thread moves per K-tile
    constexpr int B_VECS = BN * KV / NT;
    static_assert(BM * KV % NT == 0 && BN * KV % NT == 0, "tile must divide evenly over the threads");
    static_assert(NT % BN == 0 || TRANS_B, "[k,n] loader needs whole column sweeps");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T *As = reinterpret_cast<T *>(smem_raw);  // [2][BM][S]
    T *Bs = As + 2 * BM * S;                  // [2][BN][S]

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int wm0 = (wave / WN) * WTM;
    const int wn0 = (wave % WN) * WTN;

    int tile_m, tile_n;
    tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
    const int64_t batch = blockIdx.y;
    const T *A = p.a + batch * p.stride_a;
    const T *B = p.b + batch * p.stride_b;
    T *C = p.c + batch * p.stride_c;

    V a_st[A_VECS], b_st[B_VECS];

    auto load_k_contig = [&](const T *base, int64_t ld, int64_t r0, int64_t rmax, int64_t k0, V *st, auto nvecs) {
#pragma unroll
        for (int i = 0; i < decltype(nvecs)::value; ++i) {
            const int vid = tid + i * NT;
            const int row = vid / KV, kv = vid % KV;
            const int64_t gr = r0 + row, gk = k0 + kv * EPV;
            V v = M::zero();
            if (gr < rmax) {
                const T *src = base + gr * ld + gk;
                if constexpr (VEC) {
                    if (gk < p.k) v = *reinterpret_cast<const V *>(src);
                } else {
                    T e[EPV];
#pragma unroll
                    for (int j = 0; j < EPV; ++j) e[j] = (gk + j < p.k) ? src[j] : T(0);
                    v = M::make(e);
                }
            }
            st[i] = v;
        }
    };
    // B stored [k, n]: thread owns column (tid % BN) and k-vectors kv = tid / BN + i * (NT / BN).
    auto load_b_kn = [&](int64_t k0) {
        if constexpr (!TRANS_B) {
            constexpr int KV_STEP = NT / BN;
            const int col = tid % BN, kv0 = tid / BN;
            const int64_t gc = n0 + col;
#pragma unroll
            for (int i = 0; i < B_VECS; ++i) {
                const int64_t gk = k0 + (int64_t)(kv0 + i * KV_STEP) * EPV;
                T e[EPV];
#pragma unroll
                for (int j = 0; j < EPV; ++j) e[j] = (gc < p.n && gk + j < p.k) ? B[(gk + j) * p.ldb + gc] : T(0);
                b_st[i] = M::make(e);
            }
        }
    };
    auto load_tiles = [&](int64_t k0) {
        load_k_contig(A, p.lda, m0, p.m, k0, a_st, std::integral_constant<int, A_VECS>{});
        if constexpr (TRANS_B) load_k_contig(B, p.ldb, n0, p.n, k0, b_st, std::integral_constant<int, B_VECS>{});
        else load_b_kn(k0);
    };
    auto store_tiles = [&](int buf) {
        T *as = As + buf * BM * S;
        T *bs = Bs + buf * BN * S;
#pragma unroll
        for (int i = 0; i < A_VECS; ++i) {
            const int vid = tid + i * NT;
            *reinterpret_cast<V *>(as + (vid / KV) * S + (vid % KV) * EPV) = a_st[i];
        }
        if constexpr (TRANS_B) {
#pragma unroll
            for (int i = 0; i < B_VECS; ++i) {
                const int vid = tid + i * NT;
                *reinterpret_cast<V *>(bs + (vid / KV) * S + (vid % KV) * EPV) = b_st[i];
            }
        } else {
            constexpr int KV_STEP = NT / BN;
            const int col = tid % BN, kv0 = tid / BN;
#pragma unroll
            for (int i = 0; i < B_VECS; ++i) *reinterpret_cast<V *>(bs + col * S + (kv0 + i * KV_STEP) * EPV) = b_st[i];
        }
    };

    typename M::Acc acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < M::ACC; ++r) acc[i][j][r] = T(0);

    const int64_t ktiles = (p.k + BK - 1) / BK;
    const int lrow = lane % MT;           // row / column inside an MFMA tile
    const int lk = (lane / MT) * EPV;     // k offset of this lane's vector inside a fetch

    if (ktiles > 0) {
        load_tiles(0);
        store_tiles(0);
    }
    __syncthreads();

    for (int64_t kt = 0; kt < ktiles; ++kt) {
        const int buf = (int)(kt & 1);
        if (kt + 1 < ktiles) load_tiles((kt + 1) * BK);
        const T *as = As + buf * BM * S + (wm0 + lrow) * S + lk;
        const T *bs = Bs + buf * BN * S + (wn0 + lrow) * S + lk;
#pragma unroll
        for (int kc = 0; kc < BK / KCH; ++kc) {
            V af[TM], bf[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) af[i] = *reinterpret_cast<const V *>(as + i * MT * S + kc * KCH);
#pragma unroll
            for (int j = 0; j < TN; ++j) bf[j] = *reinterpret_cast<const V *>(bs + j * MT * S + kc * KCH);
#pragma unroll
            for (int e = 0; e < EPV; ++e)
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j) acc[i][j] = M::mma(M::elem(af[i], e), M::elem(bf[j], e), acc[i][j]);
        }
        if (kt + 1 < ktiles) store_tiles(buf ^ 1);
        __syncthreads();
    }

    // Epilogue: each rounding is its own step, in the order product -> alpha -> bias -> GELU ->
    // residual, which is the order the unfused reference ops would apply them.
    const bool has_bias = (p.epilogue & FTH_EPI_BIAS) != 0;
    const bool has_gelu = (p.epilogue & FTH_EPI_GELU) != 0;
    const bool has_res = (p.epilogue & FTH_EPI_RESIDUAL) != 0;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int64_t col = n0 + wn0 + j * MT + lrow;
        if (col >= p.n) continue;
        const T bv = has_bias ? p.bias[col] : T(0);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int r = 0; r < M::ACC; ++r) {
                const int64_t row = m0 + wm0 + i * MT + M::acc_row(r, lane);
                if (row < p.m) {
                    T v = acc[i][j][r];
                    if (p.use_alpha) v = p.alpha * v;
                    if (has_bias) v = v + bv;
                    if (has_gelu) v = M::gelu(v);
                    if (has_res) v = v + p.residual[batch * p.stride_c + row * p.ldc + col];
                    C[row * p.ldc + col] = v;
                }
            }
        }
    }
}

// Epilogue-only kernel for k == 0 (the product is all zeros).
template <typename T>
__global__ __launch_bounds__(256) void gemm_k0_kernel(const GemmArgs<T> p) {
    using M = Mfma<T>;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= p.m * p.n) return;
    const int64_t row = i / p.n, col = i % p.n, batch = blockIdx.y;
    T v = T(0);
    if (p.use_alpha) v = p.alpha * v;
    if (p.epilogue & FTH_EPI_BIAS) v = v + p.bias[col];
    if (p.epilogue & FTH_EPI_GELU) v = M::gelu(v);
    if (p.epilogue & FTH_EPI_RESIDUAL) v = v + p.residual[batch * p.stride_c + row * p.ldc + col];
    p.c[batch * p.stride_c + row * p.ldc + col] = v;
}

template <typename T, int BM, int BN, int BK, int WM, int WN, bool TRANS_B, bool VEC>
int32_t launch_config(GemmArgs<T> &p, int64_t batch, hipStream_t st) {
    using M = Mfma<T>;
    constexpr int S = BK + M::EPV;
    constexpr size_t smem = (size_t)2 * (BM + BN) * S * sizeof(T);
    auto kern = gemm_kernel<T, BM, BN, BK, WM, WN, TRANS_B, VEC>;
    static bool attr_set = false;  // benign race: the attribute call is idempotent
    if (!attr_set) {
        FTH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    int64_t tm = fth::ceil_div(p.m, BM), tn = fth::ceil_div(p.n, BN);
    FTH_ARG(tm * tn <= 2147483647LL && batch <= 65535, "gemm: grid too large (tiles %lld x %lld, batch %lld)",
            (long long)tm, (long long)tn, (long long)batch);
    p.tiles_m = (int)tm;
    p.tiles_n = (int)tn;
    kern<<<dim3((unsigned)(tm * tn), (unsigned)batch), dim3(WM * WN * kWave), smem, st>>>(p);
    FTH_CHECK_LAUNCH("gemm");
    return FTH_OK;
}

template <typename T, bool TRANS_B, bool VEC>
int32_t launch_shape(GemmArgs<T> &p, int64_t batch, hipStream_t st) {
    // Large problems: 128x128 tiles (2x2 wavefronts of 64x64). Problems too small to give every
    // CU a large tile: 64x64 tiles (2x2 wavefronts of 32x32).
    const int64_t big_tiles = fth::ceil_div(p.m, 128) * fth::ceil_div(p.n, 128) * batch;
    const int cus = fth::compute_units() > 0 ? fth::compute_units() : 256;
    if constexpr (std::is_same<T, float>::value) {
        if (big_tiles >= cus) return launch_config<T, 128, 128, 32, 2, 2, TRANS_B, VEC>(p, batch, st);
        return launch_config<T, 64, 64, 32, 2, 2, TRANS_B, VEC>(p, batch, st);
    } else {
        if (big_tiles >= cus) return launch_config<T, 128, 128, 16, 2, 2, TRANS_B, VEC>(p, batch, st);
        return launch_config<T, 64, 64, 16, 2, 2, TRANS_B, VEC>(p, batch, st);
    }
}

template <typename T>
int32_t gemm_entry(const fth_gemm_desc *d, T alpha, const T *a, const T *b, T *c, const T *bias, const T *residual,
                   fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(d != nullptr, "gemm: desc is NULL");
    FTH_ARG(d->m >= 0 && d->n >= 0 && d->k >= 0 && d->batch >= 0, "gemm: negative extent");
    if (d->m == 0 || d->n == 0 || d->batch == 0) return FTH_OK;  // crates/ft-kernel-cpu/src/lib.rs:1311-1313
    FTH_ARG(c != nullptr, "gemm: C is NULL");
    FTH_ARG(d->k == 0 || (a && b), "gemm: NULL operand");
    FTH_ARG(d->lda >= d->k && d->ldc >= d->n && d->ldb >= (d->trans_b ? d->k : d->n),
            "gemm: row pitch smaller than the row (lda %lld ldb %lld ldc %lld)", (long long)d->lda, (long long)d->ldb,
            (long long)d->ldc);
    FTH_ARG(!(d->epilogue & FTH_EPI_BIAS) || bias, "gemm: bias epilogue without a bias pointer");
    FTH_ARG(!(d->epilogue & FTH_EPI_RESIDUAL) || residual, "gemm: residual epilogue without a residual pointer");
    FTH_ARG((d->epilogue & ~(FTH_EPI_BIAS | FTH_EPI_GELU | FTH_EPI_RESIDUAL)) == 0, "gemm: unknown epilogue bits");
    hipStream_t st = fth::resolve_stream(s);
    GemmArgs<T> p;
    p.a = a; p.b = b; p.c = c; p.bias = bias; p.residual = residual;
    p.m = d->m; p.n = d->n; p.k = d->k;
    p.lda = d->lda; p.ldb = d->ldb; p.ldc = d->ldc;
    p.stride_a = d->stride_a; p.stride_b = d->stride_b; p.stride_c = d->stride_c;
    p.alpha = alpha;
    p.use_alpha = (alpha != T(1)) ? 1 : 0;
    p.epilogue = d->epilogue;
    p.tiles_m = p.tiles_n = 0;
    if (d->k == 0) {
        int64_t grid = fth::ceil_div(d->m * d->n, 256);
        FTH_ARG(grid <= 2147483647LL && d->batch <= 65535, "gemm: grid too large");
        gemm_k0_kernel<T><<<dim3((unsigned)grid, (unsigned)d->batch), dim3(256), 0, st>>>(p);
        FTH_CHECK_LAUNCH("gemm_k0");
        return FTH_OK;
    }
    constexpr int EPV = Mfma<T>::EPV;
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    // 128-bit global loads along k need 16-byte aligned rows in every batch.
    bool vec = d->k % EPV == 0 && d->lda % EPV == 0 && al(a) && d->stride_a % EPV == 0;
    if (d->trans_b) vec = vec && d->ldb % EPV == 0 && al(b) && d->stride_b % EPV == 0;
    if (d->trans_b) {
        return vec ? launch_shape<T, true, true>(p, d->batch, st) : launch_shape<T, true, false>(p, d->batch, st);
    }
    return vec ? launch_shape<T, false, true>(p, d->batch, st) : launch_shape<T, false, false>(p, d->batch, st);
}

}  // namespace

extern "C" {

int32_t fth_dev_gemm_f32(const fth_gemm_desc *d, float alpha, const float *a, const float *b, float *c,
                         const float *bias, const float *residual, fth_stream s) {
    return gemm_entry<float>(d, alpha, a, b, c, bias, residual, s);
}

int32_t fth_dev_gemm_f64(const fth_gemm_desc *d, double alpha, const double *a, const double *b, double *c,
                         const double *bias, const double *residual, fth_stream s) {
    return gemm_entry<double>(d, alpha, a, b, c, bias, residual, s);
}

}  // extern "C"
