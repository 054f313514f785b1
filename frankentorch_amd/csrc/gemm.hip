// Dense contraction on the gfx950 matrix cores: C = alpha * A * op(B) (+ bias, GELU, residual).
//
//   fp32: v_mfma_f32_32x32x2_f32   (32x32 output tile per wavefront instruction, k = 2)
//   fp64: v_mfma_f64_16x16x4_f64   (16x16 output tile, k = 4)
//
// Two kernels share the tiling, the schedule and the accumulation order:
//   gemm_direct_kernel  operand tiles go global -> LDS directly (global_load_lds); used whenever the
//                       operand rows are 16-byte aligned and K is a whole number of 128-byte K-tiles.
//                       Its header comment describes the LDS layout and the pipeline.
//   gemm_kernel         any K and alignment: global -> registers -> LDS, described next.
//
// Data path of gemm_kernel. A block owns a BM x BN tile of C. Both operands are staged in LDS
// K-CONTIGUOUS (As[BM][BK+pad], Bs[BN][BK+pad]), so a lane fetches its MFMA operands with one 128-bit
// LDS read: that vector holds EPV consecutive k for the lane's row, and feeds EPV successive MFMAs.
// Which k lands in which MFMA is irrelevant as long as A and B agree, and they do because both
// use the same (lane / MT, element) -> k map. The pad (one vector per row) makes the row pitch
// an odd number of vectors. Global -> LDS goes through registers, one K-tile ahead (two LDS
// buffers, one barrier per K-tile): the loads of tile t+1 are issued before the MFMAs of tile t.
//   A, and B stored [n, k] (trans_b): 128-bit global loads along k.
//   B stored [k, n]: EPV x EPV register blocks (EPV vector loads along n, regrouped in registers
//   into EPV vectors along k), or element loads when n is not a vector multiple.
//
// Scheduling. The kernel is persistent: the grid is (CUs x resident blocks per CU) workgroups,
// and the linearised iteration space (output tiles x K-tiles) is cut into equal contiguous
// ranges, one per workgroup ("stream-K"). A workgroup therefore runs whole tiles back to back
// and at most one partial tile at each end of its range; no CU idles while another still has a
// tile to finish, whatever the tile count. A tile whose K range is shared by several workgroups
// is completed without spinning, fences or atomics: every contributor writes its accumulators to
// a workspace slot, and a small second kernel (ordered after the first by the stream) adds the
// slots of each split tile in K order and runs the epilogue. The split points depend only on
// (shape, tile configuration, grid size) and the additions are in a fixed order, so results are
// bitwise repeatable on a given device.
//
// Tile order. Consecutive workgroup ids land on different XCDs (8 per device, each with its own
// L2), so the id is first remapped to give each XCD one contiguous range of the iteration space,
// and tiles are numbered in groups of GROUP_M tile-rows so that workgroups that run concurrently
// share A row-panels and B column-panels in that XCD's L2.
//
// replaces gemm::sgemm / dgemm / sgemm_bt / dgemm_bt (crates/ft-kernel-cpu/src/lib.rs:1310-1338,
// 107-138, 1430-1481, 201-255), the per-batch loop of bmm (:38572-38606) and the bias pass of
// linear_tensor_f32 (:17336-17351).

#include <cstdlib>
#include <map>
#include <mutex>
#include <type_traits>

#include "common.hpp"
#include "devmath.hpp"
#include "pool.hpp"

namespace {

constexpr int kWave = 64;
constexpr int kXcds = 8;
constexpr int kGroupM = 8;
#ifndef FTH_F32_BK
#define FTH_F32_BK 32
#endif
#ifndef FTH_EP_CHUNK
#define FTH_EP_CHUNK 0
#endif
#ifndef FTH_GD_ROTATE
#define FTH_GD_ROTATE 1
#endif
#ifndef FTH_GD_SCHED
#define FTH_GD_SCHED 1
#endif
#ifndef FTH_F32_MINW
#define FTH_F32_MINW 2
#endif

// Internal epilogue bit (not part of fth_gemm_desc.epilogue): also emit the maximum of every output row over each wavefront's
// 64 columns of the tile (GemmArgs::rowmax). fp32 direct kernel for whole tiles, the fix-up kernel for split ones.
constexpr int kEpiRowMax = 64;

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
    __device__ __forceinline__ static float gelu(float x) { return fth::gelu_erf(x); }
    // tanh-form GELU as x * sigmoid(2u), u = sqrt(2/pi) (x + 0.044715 x^3): 0.5 (1 + tanh u) = 1 / (1 + e^-2u). One
    // hardware exp2 and one division; e^-2u overflowing to inf gives x / inf = -0 where the tanh form gives -0 too.
    __device__ __forceinline__ static float gelu_tanh(float x) {
        const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
        return x / (1.0f + __builtin_amdgcn_exp2f(u * -2.8853900817779268f));  // -2 log2(e)
    }
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
    __device__ __forceinline__ static double gelu_tanh(double x) {
        return 0.5 * x * (1.0 + tanh(0.79788456080286535588 * (x + 0.044715 * x * x * x)));
    }
};

// fp32 on v_mfma_f32_16x16x4_f32: accumulator element r of `lane` is row 4 (lane / 16) + r, column lane % 16. The same
// multiply-add rate as the 32x32x2 form and the same operand traffic; measured on the products that keep a workgroup on
// one long run of tiles it is the faster of the two (8192 x 50257 x 768: 4.71 -> 4.58 ms; 4096^3 with a [n, k] B: 0.925 ->
// 0.936 of the matrix peak), on the short launches of the transformer block and on [k, m] A operands the slower one
// (linear backward 0.597 -> 0.611 ms), so it is used where DirectMfma says and nowhere else.
struct MfmaF32x16 : Mfma<float> {
    static constexpr int MT = 16;
    static constexpr int KG = 4;
    static constexpr int ACC = 4;
    using Acc = float __attribute__((ext_vector_type(4)));
    __device__ __forceinline__ static Acc mma(float a, float b, Acc c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
    __device__ __forceinline__ static int acc_row(int r, int lane) { return 4 * (lane >> 4) + r; }
};
constexpr int kEpiRowMaxBit = 64;
// The MFMA form of a direct-kernel instantiation: 16x16x4 for fp32 x . w^T on 128 x 128 tiles with no epilogue (with or
// without the row maxima), 32x32x2 (fp32) / 16x16x4 (fp64) otherwise. A function of the instantiation alone, so a shape
// always gets the same arithmetic.
template <typename T, int BM, int BN, bool TRANS_A, bool TRANS_B, int EPI> struct DirectMfma { using type = Mfma<T>; };
template <> struct DirectMfma<float, 128, 128, false, true, 0> { using type = MfmaF32x16; };
template <> struct DirectMfma<float, 128, 128, false, true, kEpiRowMaxBit> { using type = MfmaF32x16; };

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
    // persistent schedule
    int ktiles;              // K-tiles per output tile
    int64_t tiles_per_batch; // tiles_m * tiles_n
    int64_t total_iters;     // batch * tiles_per_batch * ktiles
    T *partials;             // [grid][2][BM * BN] accumulator slots of split tiles
    int grid;                // workgroups of the main kernel (the fix-up kernel needs it too)
    int order = 0;           // tile order inside a group of tile rows: 0 column-major, 1 row-major (tile_of_id)
    // Row maxima by column group (kEpiRowMax): [column groups][m], group g = columns [64 g, 64 g + 64), one wavefront's share of a tile.
    // NaN = "not known, look at the stored values" (a group with a NaN in it).
    T *rowmax = nullptr;
};

// Tile number -> (tile_m, tile_n): groups of kGroupM tile-rows; inside a group column-major (order 0: a workgroup's
// consecutive tiles share their B panel) or row-major (order 1: they share their A panel and lie side by side in the output).
// Row-major is for wide outputs, where a workgroup walks many tiles: tiles that are neighbours along a row of C share the
// 128-byte lines at their common edge whenever the row pitch is not a multiple of 128 bytes (the [8192, 50257] logits), and
// written a tile apart in time by one workgroup those lines are completed in cache; written 8 tiles apart, as in order 0,
// they leave as two partial writes. Measured on the LM head: 4.83 -> 4.75 ms (4.63 -> 4.59 ms at an aligned pitch of 50304);
// the square 4096^3 product, two tiles per workgroup, is 0.3 % better in order 0.
__device__ __forceinline__ void tile_of_id(int64_t id, int tiles_m, int tiles_n, int &tm, int &tn, int order) {
    const int64_t group = (int64_t)kGroupM * tiles_n;
    const int64_t g = id / group;
    const int first_m = (int)(g * kGroupM);
    const int gm = (tiles_m - first_m) < kGroupM ? (tiles_m - first_m) : kGroupM;
    const int in_g = (int)(id - g * group);
    if (order == 1) {
        tm = first_m + in_g / tiles_n;
        tn = in_g % tiles_n;
        return;
    }
    tm = first_m + in_g % gm;
    tn = in_g / gm;
}

// Hardware workgroup id -> virtual id such that each XCD owns one contiguous run of virtual ids.
__device__ __forceinline__ int xcd_contiguous_id(int pid, int grid) {
    const int per = grid / kXcds, rem = grid % kXcds;
    const int xcd = pid % kXcds, q = pid / kXcds;
    return q + xcd * per + (xcd < rem ? xcd : rem);
}

// VEC:  128-bit global loads along k are legal for A (and for B when it is stored [n, k]).
// VECB: B is stored [k, n] and 128-bit global loads along n are legal; the loader then moves
//       EPV x EPV register blocks (EPV vector loads, transposed in registers, EPV vector LDS stores).
template <typename T, int BM, int BN, int BK, int WM, int WN, int MINW, bool TRANS_B, bool VEC, bool VECB>
__global__ __launch_bounds__(WM *WN *kWave, MINW) void gemm_kernel(const GemmArgs<T> p) {
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
    // Register-block loader for [k, n] B: the tile holds B_BLOCKS blocks of EPV x EPV elements,
    // B_BPT per thread (threads past the last block of a sweep carry none).
    constexpr int B_BLOCKS = KV * (BN / EPV);
    constexpr int B_BPT = (B_BLOCKS + NT - 1) / NT;
    constexpr bool BLOCK_B = !TRANS_B && VECB && (NT % (BN / EPV) == 0);
    constexpr int B_ST = BLOCK_B ? B_BPT * EPV : B_VECS;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T *As = reinterpret_cast<T *>(smem_raw);  // [2][BM][S]
    T *Bs = As + 2 * BM * S;                  // [2][BN][S]

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int wm0 = (wave / WN) * WTM;
    const int wn0 = (wave % WN) * WTN;

    // Per-segment state (set at the top of the persistent loop; the loaders read it by reference).
    int64_t m0 = 0, n0 = 0, batch = 0;
    const T *A = p.a;
    const T *B = p.b;
    T *C = p.c;

    V a_st[A_VECS], b_st[B_ST];

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
    // B stored [k, n], register-block form: thread owns EPV consecutive columns (4 * nv) and
    // k-vectors kq = tid / (BN / EPV) + blk * (NT / (BN / EPV)); it loads EPV rows of EPV columns
    // and regroups them into EPV vectors of EPV consecutive k, one per column.
    auto load_b_blocks = [&](int64_t k0) {
        if constexpr (BLOCK_B) {
            constexpr int NV = BN / EPV, KQ_STEP = NT / NV;
            const int nv = tid % NV, kq0 = tid / NV;
            const int64_t gc = n0 + (int64_t)nv * EPV;
#pragma unroll
            for (int blk = 0; blk < B_BPT; ++blk) {
                const int kq = kq0 + blk * KQ_STEP;
                const int64_t gk = k0 + (int64_t)kq * EPV;
                V rows[EPV];
#pragma unroll
                for (int j = 0; j < EPV; ++j) {
                    // n % EPV == 0 and k % EPV == 0 are guaranteed by the launcher for this path
                    rows[j] = (kq < KV && gc < p.n && gk + j < p.k) ? *reinterpret_cast<const V *>(B + (gk + j) * p.ldb + gc) : M::zero();
                }
#pragma unroll
                for (int c = 0; c < EPV; ++c) {
                    T e[EPV];
#pragma unroll
                    for (int j = 0; j < EPV; ++j) e[j] = M::elem(rows[j], c);
                    b_st[blk * EPV + c] = M::make(e);
                }
            }
        }
    };
    // B stored [k, n], scalar form: thread owns column (tid % BN) and k-vectors kv = tid / BN + i * (NT / BN).
    auto load_b_kn = [&](int64_t k0) {
        if constexpr (!TRANS_B && !BLOCK_B) {
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
        else if constexpr (BLOCK_B) load_b_blocks(k0);
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
        } else if constexpr (BLOCK_B) {
            constexpr int NV = BN / EPV, KQ_STEP = NT / NV;
            const int nv = tid % NV, kq0 = tid / NV;
#pragma unroll
            for (int blk = 0; blk < B_BPT; ++blk) {
                const int kq = kq0 + blk * KQ_STEP;
                if (kq < KV) {
#pragma unroll
                    for (int c = 0; c < EPV; ++c) *reinterpret_cast<V *>(bs + (nv * EPV + c) * S + kq * EPV) = b_st[blk * EPV + c];
                }
            }
        } else {
            constexpr int KV_STEP = NT / BN;
            const int col = tid % BN, kv0 = tid / BN;
#pragma unroll
            for (int i = 0; i < B_VECS; ++i) *reinterpret_cast<V *>(bs + col * S + (kv0 + i * KV_STEP) * EPV) = b_st[i];
        }
    };

    typename M::Acc acc[TM][TN];
    const int lrow = lane % MT;           // row / column inside an MFMA tile
    const int lk = (lane / MT) * EPV;     // k offset of this lane's vector inside a fetch

    // Epilogue: each rounding is its own step, in the order product -> alpha -> bias -> GELU ->
    // residual, which is the order the unfused reference ops would apply them.
    const bool has_bias = (p.epilogue & FTH_EPI_BIAS) != 0;
    const bool has_gelu = (p.epilogue & FTH_EPI_GELU) != 0;
    const bool has_gelu_tanh = (p.epilogue & FTH_EPI_GELU_TANH) != 0;
    const bool has_res = (p.epilogue & FTH_EPI_RESIDUAL) != 0;
    auto epilogue = [&]() {
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
                        if (has_gelu_tanh) v = M::gelu_tanh(v);
                        if (has_res) v = v + p.residual[batch * p.stride_c + row * p.ldc + col];
                        C[row * p.ldc + col] = v;
                    }
                }
            }
        }
    };

    const int grid = (int)gridDim.x;
    const int vb = xcd_contiguous_id((int)blockIdx.x, grid);
    const int64_t total = p.total_iters;
    // Workgroup b owns iterations [b * total / grid, (b + 1) * total / grid).
    int64_t it = (int64_t)vb * total / grid;
    const int64_t it_end = (int64_t)(vb + 1) * total / grid;

    while (it < it_end) {
        const int64_t tile = it / p.ktiles;
        const int k_lo = (int)(it - tile * p.ktiles);
        const int64_t left = it_end - it;
        const int nk = (int)((int64_t)(p.ktiles - k_lo) < left ? (int64_t)(p.ktiles - k_lo) : left);
        batch = tile / p.tiles_per_batch;
        int tile_m, tile_n;
        tile_of_id(tile - batch * p.tiles_per_batch, p.tiles_m, p.tiles_n, tile_m, tile_n, p.order);
        m0 = (int64_t)tile_m * BM;
        n0 = (int64_t)tile_n * BN;
        A = p.a + batch * p.stride_a;
        B = p.b + batch * p.stride_b;
        C = p.c + batch * p.stride_c;

#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < M::ACC; ++r) acc[i][j][r] = T(0);

        load_tiles((int64_t)k_lo * BK);
        store_tiles(0);
        __syncthreads();
        for (int kt = 0; kt < nk; ++kt) {
            const int buf = kt & 1;
            if (kt + 1 < nk) load_tiles((int64_t)(k_lo + kt + 1) * BK);
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
            if (kt + 1 < nk) store_tiles(buf ^ 1);
            __syncthreads();
        }

        if (nk == p.ktiles) {
            epilogue();
        } else {
            // Split tile: park the accumulators; gemm_fixup_kernel adds the contributions in K order.
            // Slot layout: the thread's TM * TN * ACC values in flat order e, as 16-byte vectors
            // interleaved over the threads ([e / EPV][tid][e % EPV]), so both sides move whole vectors.
            constexpr int64_t SLOT = (int64_t)BM * BN;
            T *mine = p.partials + ((int64_t)vb * 2 + (k_lo > 0 ? 0 : 1)) * SLOT;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int r = 0; r < M::ACC; r += EPV) {
                        T e[EPV];
#pragma unroll
                        for (int q = 0; q < EPV; ++q) e[q] = acc[i][j][r + q];
                        const int ev = ((i * TN + j) * M::ACC + r) / EPV;
                        *reinterpret_cast<V *>(mine + ((int64_t)ev * NT + tid) * EPV) = M::make(e);
                    }
        }
        it += nk;
    }
}

// ---- direct-to-LDS variant (A [m,k] with 16-byte aligned rows; B stored [n,k] or [k,n]) ----
//
// Same tiling, schedule, accumulation order and slot format as gemm_kernel; only the way operand
// tiles reach LDS and the LDS layout differ. A K-tile is 128 bytes of k per row (32 floats, 16
// doubles). Tiles are written by global_load_lds (16 bytes per lane, no staging registers and no
// LDS store instructions): one wavefront instruction fills 1 KiB of LDS in lane order.
//   k-contiguous operands (A, and B stored [n,k]): a chunk is 8 rows x 8 vectors, unpadded. To
//   keep the MFMA operand reads conflict-free the vectors of a row are stored XOR-swizzled:
//   logical vector q of row r sits in slot q ^ ((r >> 1) & 7). The loader does the swizzle on the
//   global side (lane -> slot is fixed by the hardware, so lane (r, slot) fetches vector
//   slot ^ ((r >> 1) & 7) of its row); the 8 lanes of a row still cover one whole 128-byte line.
//   B stored [k,n]: the tile is kept [k][n] as it is in memory (a chunk is 1 KiB of consecutive
//   n of one or more k rows) and a lane reads its MFMA operand element by element; consecutive
//   lanes read consecutive n, which is conflict-free without padding.
// Rows (columns) past the m / n edge are clamped to the last valid one: a row of A (column of B)
// only feeds the same row (column) of C, and those are never stored. The launcher guarantees
// k % BK == 0. The loader runs one K-tile ahead of the MFMAs across output-tile boundaries too,
// so the first K-tile of the next output tile is in flight during the epilogue of this one.
// Calls f(integral_constant<int, 0>{}) ... f(integral_constant<int, N - 1>{}).
template <int N, int I = 0, typename F> __device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<N, I + 1>(f);
    }
}

// A pointer every lane holds the same value of, made a scalar for the compiler (two v_readfirstlane_b32 where it
// had the value in vector registers, nothing where it was scalar already).
template <typename T> __device__ __forceinline__ const T *uniform_ptr(const T *ptr) {
    const uint64_t v = reinterpret_cast<uint64_t>(ptr);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<const T *>(((uint64_t)hi << 32) | lo);
}

template <typename T> __device__ __forceinline__ void load_to_lds_16(const T *base, unsigned lane_bytes, unsigned lds_chunk) {
    // Inline assembly so that the compiler's wait-count insertion does not see an LDS write it
    // cannot disambiguate (it would drain the load queue before every LDS read and serialise the
    // prefetch); the kernel waits for vmcnt(0) itself before each barrier.
    // Scalar base (the K-tile's uniform pointer) plus a per-lane 32-bit byte offset: no 64-bit vector address
    // arithmetic per load (vector instructions take issue cycles from the MFMAs). The chunk address is the same in
    // every lane; readfirstlane makes that explicit so the operand is an SGPR.
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_bytes), "s"(base),
                 "s"(__builtin_amdgcn_readfirstlane(lds_chunk))
                 : "memory", "m0");
}

// ---- row maxima of a wavefront's share of a tile (kEpiRowMax, 16 x 16 accumulators) ----
// A lane holds four consecutive rows of ONE column of each 16 x 16 accumulator, and a wavefront's 64 columns of a row block
// are four accumulators side by side, so the four are combined in the lane first; what is left is a reduction over the 16
// lanes of a DPP row (the lanes that share lane / 16, i.e. the same four rows). It is done as a transposing butterfly over
// the quad -- a lane keeps two of its four rows and hands the other two to lane ^ 1, then one of two to lane ^ 2 -- followed
// by two row rotations (by 4 and by 8 lanes) that combine the four quads: 3 + 2 exchanges instead of 4 x 4. Lane l ends up
// with the maximum of row element rowmax_elem_of_lane(l) over the wavefront's 64 columns.
// The maximum is the NaN-propagating one (v_maximum3_f32): a group with a NaN in it comes out as NaN, which is exactly the
// "not known, look at the stored values" marker the consumer expects, and +-inf are ordinary values.
template <int CTRL> __device__ __forceinline__ float dpp_take(float x) {
    const int xi = __builtin_bit_cast(int, x);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(xi, xi, CTRL, 0xF, 0xF, false));
}
__device__ __forceinline__ float nan_max(float a, float b) { return __builtin_elementwise_maximum(a, b); }
__device__ __forceinline__ float rowmax_fold(float (&v)[4], int lane) {
    constexpr int kRor4 = 0x124, kRor8 = 0x128, kXor1 = 0xB1, kXor2 = 0x4E;  // row_ror:4, row_ror:8, quad_perm [1,0,3,2], [2,3,0,1]
    const bool up1 = (lane & 1) != 0, up2 = (lane & 2) != 0;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const float keep = up1 ? v[k + 2] : v[k], send = up1 ? v[k] : v[k + 2];
        v[k] = nan_max(keep, dpp_take<kXor1>(send));
    }
    const float keep = up2 ? v[1] : v[0], send = up2 ? v[0] : v[1];
    float m = nan_max(keep, dpp_take<kXor2>(send));
    m = nan_max(m, dpp_take<kRor4>(m));
    return nan_max(m, dpp_take<kRor8>(m));
}
__device__ __forceinline__ int rowmax_elem_of_lane(int lane) { return ((lane & 1) << 1) | ((lane >> 1) & 1); }

// EPI >= 0: the epilogue flags are this compile-time mask and alpha is 1 (straight-line output code);
// EPI < 0: flags and alpha are read from the arguments.
// TRANS_A: A is stored [k, m] (its tile is kept [k][m] in LDS and read element-wise, like a [k,n] B).
template <typename T, int BM, int BN, int WM, int WN, int MINW, bool TRANS_A, bool TRANS_B, int EPI>
__global__ __launch_bounds__(WM *WN *kWave, MINW) void gemm_direct_kernel(const GemmArgs<T> p) {
    using M = typename DirectMfma<T, BM, BN, TRANS_A, TRANS_B, EPI>::type;
    using V = typename M::V;
    constexpr int MT = M::MT, KG = M::KG, EPV = M::EPV;
    constexpr int NW = WM * WN, NT = NW * kWave;
    constexpr int BK = 128 / (int)sizeof(T);
    constexpr int KCH = KG * EPV, NCH = BK / KCH;
    constexpr int WTM = BM / WM, WTN = BN / WN;
    constexpr int TM = WTM / MT, TN = WTN / MT;
    constexpr int A_LD = BM / 8 / NW;                         // chunk loads per wavefront and K-tile
    constexpr int B_LD = BN * BK * (int)sizeof(T) / 1024 / NW;
    constexpr int LPR = BN * (int)sizeof(T) / 16;             // [k,n] B: lanes per k row of the tile
    constexpr int RPC = kWave / LPR;                          // [k,n] B: k rows per chunk
    constexpr int LPR_A = BM * (int)sizeof(T) / 16;           // [k,m] A: the same for A
    constexpr int RPC_A = kWave / LPR_A;
    static_assert(LPR_A <= kWave && kWave % LPR_A == 0, "a chunk must hold whole k rows of A");
    static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "tile rows must divide into 8-row chunks per wavefront");
    static_assert(MT % 16 == 0, "swizzle assumes MFMA tile rows start on a multiple of 16");
    // [k,n] B: chunks of whole k rows where a row's vectors divide the wavefront (BN = 64, 128); otherwise (BN = 96: 24
    // vectors a row) the tile's vectors are dealt to the lanes in row-major order and a chunk ends mid-row.
    constexpr bool B_WHOLE_ROWS = LPR <= kWave && kWave % LPR == 0;
    static_assert(TRANS_B || B_WHOLE_ROWS || BK * LPR % kWave == 0, "the [k,n] tile must be a whole number of chunks");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T *As = reinterpret_cast<T *>(smem_raw);  // [2][BM][BK]
    T *Bs = As + 2 * BM * BK;                 // [2][BN][BK] or [2][BK][BN]

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int wm0 = (wave / WN) * WTM;
    const int wn0 = (wave % WN) * WTN;
    const int lrow = lane % MT;
    // low half of a flat LDS address = LDS offset
    const unsigned lds0 = __builtin_amdgcn_readfirstlane((unsigned)reinterpret_cast<uintptr_t>(smem_raw));
    const unsigned wave_u = __builtin_amdgcn_readfirstlane((unsigned)wave);
    const int lr = lane >> 3;                           // loader: row inside the chunk
    // Swizzle term of tile row r. The LDS serves a 128-bit read 16 lanes at a time over 64 banks
    // (256 bytes), so 16 consecutive rows at the same logical vector must differ in
    // (row parity, slot): slot = q ^ ((r >> 1) & 7).
    auto swz = [](int r) __attribute__((always_inline)) { return (r >> 1) & 7; };
    // loader: k offset of the vector this lane fetches for 8-row chunk c of the tile
    auto lvec = [&](int c) __attribute__((always_inline)) { return ((lane & 7) ^ swz(c * 8 + lr)) * EPV; };
    int roff[NCH];                                      // reader: swizzled k offset per operand fetch
#pragma unroll
    for (int kc = 0; kc < NCH; ++kc) roff[kc] = ((kc * KG + lane / MT) ^ swz(lrow)) * EPV;

    constexpr bool ROWMAX = EPI >= 0 && (EPI & kEpiRowMax) != 0 && std::is_same<T, float>::value;
    static_assert(kEpiRowMax == kEpiRowMaxBit, "one bit, two names");
    const int epi = EPI >= 0 ? (EPI & ~kEpiRowMax) : p.epilogue;
    const bool has_bias = (epi & FTH_EPI_BIAS) != 0;
    const bool has_gelu = (epi & FTH_EPI_GELU) != 0;
    const bool has_gelu_tanh = (epi & FTH_EPI_GELU_TANH) != 0;
    const bool has_res = (epi & FTH_EPI_RESIDUAL) != 0;
    const bool use_alpha = EPI >= 0 ? false : p.use_alpha != 0;

    const int grid = (int)gridDim.x;
    const int vb = xcd_contiguous_id((int)blockIdx.x, grid);
    const int64_t total = p.total_iters;
    int64_t it = (int64_t)vb * total / grid;
    const int64_t it_end = (int64_t)(vb + 1) * total / grid;
    if (it >= it_end) return;

    // ---- loader state: runs one K-tile ahead of the MFMAs ----
    int n_iter = (int)(it_end - it);  // K-tiles this workgroup still has to multiply (fits: launcher check)
    int ld_left = n_iter;             // K-tiles it still has to request
    int64_t ld_tile = it / p.ktiles;
    int ld_k = (int)(it - ld_tile * p.ktiles);
    const T *ak = nullptr, *bk = nullptr;  // uniform bases of the next K-tile to load
    unsigned a_off[A_LD], b_off[B_LD];     // per-lane BYTE offsets from them; they fit 32 bits (launcher check)
    auto setup_loader = [&]() __attribute__((always_inline)) {
        const int64_t batch = ld_tile / p.tiles_per_batch;
        int tile_m, tile_n;
        tile_of_id(ld_tile - batch * p.tiles_per_batch, p.tiles_m, p.tiles_n, tile_m, tile_n, p.order);
        const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
        const int a_rows = (int)((p.m - m0) < BM ? (p.m - m0) : BM), b_cols = (int)((p.n - n0) < BN ? (p.n - n0) : BN);
        if constexpr (!TRANS_A) {
            ak = uniform_ptr(p.a + batch * p.stride_a + m0 * p.lda + (int64_t)ld_k * BK);
#pragma unroll
            for (int i = 0; i < A_LD; ++i) {
                int row = (wave * A_LD + i) * 8 + lr;
                row = row < a_rows ? row : a_rows - 1;
                a_off[i] = ((unsigned)row * (unsigned)p.lda + (unsigned)lvec(wave * A_LD + i)) * (unsigned)sizeof(T);
            }
        } else {
            ak = uniform_ptr(p.a + batch * p.stride_a + (int64_t)ld_k * BK * p.lda + m0);
            int col = (lane % LPR_A) * EPV;
            col = col < a_rows ? col : a_rows - EPV;  // m is a multiple of EPV on this path
#pragma unroll
            for (int i = 0; i < A_LD; ++i) {
                const int krow = (wave * A_LD + i) * RPC_A + lane / LPR_A;
                a_off[i] = ((unsigned)krow * (unsigned)p.lda + (unsigned)col) * (unsigned)sizeof(T);
            }
        }
        if constexpr (TRANS_B) {
            bk = uniform_ptr(p.b + batch * p.stride_b + n0 * p.ldb + (int64_t)ld_k * BK);
#pragma unroll
            for (int i = 0; i < B_LD; ++i) {
                int row = (wave * B_LD + i) * 8 + lr;
                row = row < b_cols ? row : b_cols - 1;
                b_off[i] = ((unsigned)row * (unsigned)p.ldb + (unsigned)lvec(wave * B_LD + i)) * (unsigned)sizeof(T);
            }
        } else {
            bk = uniform_ptr(p.b + batch * p.stride_b + (int64_t)ld_k * BK * p.ldb + n0);
            if constexpr (B_WHOLE_ROWS) {
                int col = (lane % LPR) * EPV;
                col = col < b_cols ? col : b_cols - EPV;  // n is a multiple of EPV on this path
#pragma unroll
                for (int i = 0; i < B_LD; ++i) {
                    const int krow = (wave * B_LD + i) * RPC + lane / LPR;
                    b_off[i] = ((unsigned)krow * (unsigned)p.ldb + (unsigned)col) * (unsigned)sizeof(T);
                }
            } else {
#pragma unroll
                for (int i = 0; i < B_LD; ++i) {
                    const int vec = (wave * B_LD + i) * kWave + lane;  // vector index in the [BK][LPR] tile
                    const int krow = vec / LPR;
                    int col = (vec % LPR) * EPV;
                    col = col < b_cols ? col : b_cols - EPV;
                    b_off[i] = ((unsigned)krow * (unsigned)p.ldb + (unsigned)col) * (unsigned)sizeof(T);
                }
            }
        }
    };
    auto issue = [&](int buf) __attribute__((always_inline)) {
        // LDS byte offsets of this wavefront's chunks (wavefront-uniform scalars)
        const unsigned as = lds0 + (unsigned)(buf * BM * BK * (int)sizeof(T)) + wave_u * (A_LD * 1024u);
        const unsigned bs = lds0 + (unsigned)((2 * BM + buf * BN) * BK * (int)sizeof(T)) + wave_u * (B_LD * 1024u);
#pragma unroll
        for (int i = 0; i < A_LD; ++i) load_to_lds_16(ak, a_off[i], as + i * 1024u);
#pragma unroll
        for (int i = 0; i < B_LD; ++i) load_to_lds_16(bk, b_off[i], bs + i * 1024u);
        ak += TRANS_A ? (int64_t)BK * p.lda : (int64_t)BK;
        bk += TRANS_B ? (int64_t)BK : (int64_t)BK * p.ldb;
        --ld_left;
        if (++ld_k == p.ktiles) {
            ld_k = 0;
            ++ld_tile;
            if (ld_left > 0) setup_loader();  // the next load starts a new output tile
        }
    };

    // ---- operand fetch: LDS -> registers, one k-chunk ahead of the MFMAs (two register slots) ----
    T af[2][TM][EPV], bf[2][TN][EPV];
    auto fetch = [&](int buf, int kc, int slot) __attribute__((always_inline)) {
        // Operand base of this lane: row (w0 + lrow) of a k-contiguous [rows][k] tile, or column
        // (w0 + lrow) and k row (lane / MT) * EPV of a [k][rows] tile.
        const T *as = !TRANS_A ? As + buf * BM * BK + (wm0 + lrow) * BK : As + buf * BK * BM + (lane / MT) * EPV * BM + wm0 + lrow;
        const T *bs = TRANS_B ? Bs + buf * BN * BK + (wn0 + lrow) * BK : Bs + buf * BK * BN + (lane / MT) * EPV * BN + wn0 + lrow;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            if constexpr (!TRANS_A) {
                const V v = *reinterpret_cast<const V *>(as + i * MT * BK + roff[kc]);
#pragma unroll
                for (int e = 0; e < EPV; ++e) af[slot][i][e] = M::elem(v, e);
            } else {
#pragma unroll
                for (int e = 0; e < EPV; ++e) af[slot][i][e] = as[(kc * KCH + e) * BM + i * MT];
            }
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            if constexpr (TRANS_B) {
                const V v = *reinterpret_cast<const V *>(bs + j * MT * BK + roff[kc]);
#pragma unroll
                for (int e = 0; e < EPV; ++e) bf[slot][j][e] = M::elem(v, e);
            } else {
#pragma unroll
                for (int e = 0; e < EPV; ++e) bf[slot][j][e] = bs[(kc * KCH + e) * BN + j * MT];
            }
        }
    };
    static_assert(NCH % 2 == 0, "the register slot of chunk 0 must be the same in every K-tile");
    // Pinning the source order (operand reads of chunk c + 1 ahead of the MFMAs of chunk c) pays for
    // fp64, whose 16x16x4 MFMAs leave little room behind them; for fp32 the compiler's own placement
    // (reads a few MFMAs before the end of a chunk) measures faster.
    constexpr bool kRotate = FTH_GD_ROTATE != 0, kSched = FTH_GD_SCHED != 0 && std::is_same<T, double>::value;

    setup_loader();
    issue(0);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wavefront's tile parts have landed
    __syncthreads();
    int cbuf = 0;
    if constexpr (kRotate) fetch(0, 0, 0);

    typename M::Acc acc[TM][TN];

    // ---- output stage ----
    // out_part<s>(src, ...) finishes one share (PARTS shares per tile) of a tile's accumulators:
    // the epilogue and the store to C for a whole tile, or the park into this workgroup's slot for a
    // split tile. With DEFER the finished tile's accumulators are copied to `old` and the shares are
    // written during the first PARTS K-tiles of the next tile: the stores are spread in time instead
    // of arriving from every workgroup at once, and their VALU work sits between that tile's MFMAs.
    constexpr bool DEFER = std::is_same<T, float>::value && kRotate;
    constexpr int PARTS = TM * TN >= 4 ? 4 : TM * TN;
    constexpr int TILES_PP = TM * TN / PARTS;  // MFMA tiles per share
    static_assert(TM * TN % PARTS == 0, "shares must be whole MFMA tiles");
    typename M::Acc old[DEFER ? TM : 1][DEFER ? TN : 1];
    bool pend = false, pend_full = false;
    int64_t pm0 = 0, pn0 = 0, pbatch = 0;
    T *pslot = nullptr;
    T res[DEFER ? TILES_PP : 1][DEFER ? M::ACC : 1];  // residual values of the share being written
    T bias_v[DEFER ? TILES_PP : 1];

    // Interior tiles (no m / n edge inside) address C and the residual as a wavefront-uniform row
    // base plus one per-lane offset: acc_row(r, lane) = acc_row(r, 0) + acc_row(0, lane), so the r
    // term moves into the scalar base and every store is `base[lane_off]` with no bounds test.
    const unsigned lane_off = (unsigned)M::acc_row(0, lane) * (unsigned)p.ldc + (unsigned)lrow;
    auto is_interior = [&](int64_t m0_, int64_t n0_) __attribute__((always_inline)) { return m0_ + BM <= p.m && n0_ + BN <= p.n; };

    // Loads the bias and residual values a share needs (ahead of the K-tile loads of the iteration
    // that will use them, so that waiting for them does not wait for those).
    auto out_load = [&](auto S, bool full, int64_t m0_, int64_t n0_, int64_t batch_) __attribute__((always_inline)) {
        constexpr int sidx = decltype(S)::value;
        if (!DEFER || !full || !(has_bias || has_res)) return;
        const bool interior = is_interior(m0_, n0_);
#pragma unroll
        for (int u = 0; u < TILES_PP; ++u) {
            const int t = sidx * TILES_PP + u, i = t / TN, j = t % TN;
            const int64_t col = n0_ + wn0 + j * MT + lrow;
            bias_v[u] = (has_bias && col < p.n) ? p.bias[col] : T(0);
            if (has_res) {
                if (interior) {
                    const T *rb = p.residual + batch_ * p.stride_c + (m0_ + wm0 + i * MT) * p.ldc + (n0_ + wn0 + j * MT);
#pragma unroll
                    for (int r = 0; r < M::ACC; ++r) res[u][r] = (rb + (int64_t)M::acc_row(r, 0) * p.ldc)[lane_off];
                } else {
#pragma unroll
                    for (int r = 0; r < M::ACC; ++r) {
                        const int64_t row = m0_ + wm0 + i * MT + M::acc_row(r, lane);
                        res[u][r] = (col < p.n && row < p.m) ? p.residual[batch_ * p.stride_c + row * p.ldc + col] : T(0);
                    }
                }
            }
        }
    };
    auto finish = [&](T v, T bv, T rv) __attribute__((always_inline)) {
        if (use_alpha) v = p.alpha * v;
        if (has_bias) v = v + bv;
        if (has_gelu) v = M::gelu(v);
        if (has_gelu_tanh) v = M::gelu_tanh(v);
        if (has_res) v = v + rv;
        return v;
    };
    // Row block i of a whole tile has been written (its TN accumulators side by side, combined in `v`): one maximum per row
    // over this wavefront's 64 columns, from the lanes that hold it after the fold.
    auto rowmax_emit = [&](float (&v)[4], int i, int64_t m0_, int64_t n0_) __attribute__((always_inline)) {
        const float mine = rowmax_fold(v, lane);
        const int64_t row = m0_ + wm0 + i * MT + M::acc_row(rowmax_elem_of_lane(lane), lane);
        const int64_t group = (n0_ + wn0) / WTN;
        if ((lane & 15) < 4 && row < p.m) p.rowmax[group * p.m + row] = mine;
    };
    auto out_store = [&](auto S, auto &src, bool full, int64_t m0_, int64_t n0_, int64_t batch_, T *slot_) __attribute__((always_inline)) {
        constexpr int sidx = decltype(S)::value;
        if (full) {
            const bool interior = is_interior(m0_, n0_);
            // Row maxima: a share is one row block of the wavefront's part of the tile (its TN accumulators side by side).
            static_assert(!ROWMAX || (M::ACC == 4 && TILES_PP == TN), "the row-maximum epilogue is written for 16 x 16 accumulators");
            float seen[ROWMAX ? 4 : 1];  // per accumulator row: the largest value written, -inf where this lane wrote none
            if constexpr (ROWMAX) {
#pragma unroll
                for (int r = 0; r < 4; ++r) seen[r] = -__builtin_inff();
            }
#pragma unroll
            for (int u = 0; u < TILES_PP; ++u) {
                const int t = sidx * TILES_PP + u, i = t / TN, j = t % TN;
                const int64_t col = n0_ + wn0 + j * MT + lrow;
                auto note = [&](int r, T val) __attribute__((always_inline)) {
                    if constexpr (ROWMAX) seen[r] = nan_max(seen[r], (float)val);
                };
                if (interior) {
                    const int64_t tile_off = batch_ * p.stride_c + (m0_ + wm0 + i * MT) * p.ldc + (n0_ + wn0 + j * MT);
                    T *cb = p.c + tile_off;
                    const T bv = DEFER ? bias_v[u] : (has_bias ? p.bias[col] : T(0));
#pragma unroll
                    for (int r = 0; r < M::ACC; ++r) {
                        const int64_t row_off = (int64_t)M::acc_row(r, 0) * p.ldc;
                        const T rv = !has_res ? T(0) : DEFER ? res[u][r] : (p.residual + tile_off + row_off)[lane_off];
                        const T val = finish(src[i][j][r], bv, rv);
                        (cb + row_off)[lane_off] = val;
                        note(r, val);
                    }
                } else if (col < p.n) {
                    T *C = p.c + batch_ * p.stride_c;
                    const T bv = DEFER ? bias_v[u] : (has_bias ? p.bias[col] : T(0));
#pragma unroll
                    for (int r = 0; r < M::ACC; ++r) {
                        const int64_t row = m0_ + wm0 + i * MT + M::acc_row(r, lane);
                        if (row < p.m) {
                            const T rv = !has_res ? T(0) : DEFER ? res[u][r] : p.residual[batch_ * p.stride_c + row * p.ldc + col];
                            const T val = finish(src[i][j][r], bv, rv);
                            C[row * p.ldc + col] = val;
                            note(r, val);
                        }
                    }
                }
            }
            if constexpr (ROWMAX) rowmax_emit(seen, sidx * TILES_PP / TN, m0_, n0_);
        } else {
#pragma unroll
            for (int u = 0; u < TILES_PP; ++u) {
                const int t = sidx * TILES_PP + u, i = t / TN, j = t % TN;
#pragma unroll
                for (int r = 0; r < M::ACC; r += EPV) {
                    T e[EPV];
#pragma unroll
                    for (int q = 0; q < EPV; ++q) e[q] = src[i][j][r + q];
                    const int ev = ((i * TN + j) * M::ACC + r) / EPV;
                    *reinterpret_cast<V *>(slot_ + ((int64_t)ev * NT + tid) * EPV) = M::make(e);
                }
            }
        }
    };

    // One K-tile: request the next one, multiply this one. EP >= 0 also writes share EP of `old`.
    auto k_iteration = [&](auto EP) __attribute__((always_inline)) {
        constexpr int ep = decltype(EP)::value;
        if constexpr (ep >= 0) out_load(EP, pend_full, pm0, pn0, pbatch);
        if (ld_left > 0) issue(cbuf ^ 1);
        if constexpr (!kRotate) fetch(cbuf, 0, 0);
#pragma unroll
        for (int kc = 0; kc < NCH; ++kc) {
            const int cur = kc & 1;
            if (kc + 1 < NCH) {
                fetch(cbuf, kc + 1, cur ^ 1);
            } else if constexpr (kRotate) {
                // Last chunk: its operands are already in registers. Close the K-tile (own loads
                // landed, everyone done reading this buffer) and fetch the first chunk of the next
                // K-tile before this chunk's MFMAs, so the matrix pipe never waits on LDS latency.
                __builtin_amdgcn_s_waitcnt(0x0F70);
                __syncthreads();
                cbuf ^= 1;
                if (--n_iter > 0) fetch(cbuf, 0, 0);
            }
            if constexpr (kSched) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int e = 0; e < EPV; ++e)
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j) acc[i][j] = M::mma(af[cur][i][e], bf[cur][j][e], acc[i][j]);
            if constexpr (kSched) __builtin_amdgcn_sched_barrier(0);
            if constexpr (!kSched && !TRANS_B) {
                // [k,n] B: spread the next chunk's operand reads over the second half of this
                // chunk's MFMAs (measured 2 % faster than the compiler's own placement).
                __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                }
            }
            if constexpr (ep >= 0) {
                if (kc == FTH_EP_CHUNK) out_store(EP, old, pend_full, pm0, pn0, pbatch, pslot);
            }
        }
        if constexpr (!kRotate) {
            __builtin_amdgcn_s_waitcnt(0x0F70);
            __syncthreads();
            cbuf ^= 1;
            --n_iter;
        }
    };
    using NoEp = std::integral_constant<int, -1>;

    while (n_iter > 0) {
        const int64_t tile = it / p.ktiles;
        const int k_lo = (int)(it - tile * p.ktiles);
        const int nk = (p.ktiles - k_lo) < n_iter ? (p.ktiles - k_lo) : n_iter;
        const int64_t batch = tile / p.tiles_per_batch;
        int tile_m, tile_n;
        tile_of_id(tile - batch * p.tiles_per_batch, p.tiles_m, p.tiles_n, tile_m, tile_n, p.order);
        const int64_t m0 = (int64_t)tile_m * BM;
        const int64_t n0 = (int64_t)tile_n * BN;

#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < M::ACC; ++r) acc[i][j][r] = T(0);

        int kt = 0;
        if constexpr (DEFER) {
            if (pend) {
                // Write the previous tile, one share per K-tile of this one (bare if this segment is shorter).
                auto step = [&](auto S) __attribute__((always_inline)) {
                    if (kt < nk) {
                        k_iteration(S);
                        ++kt;
                    } else {
                        out_load(S, pend_full, pm0, pn0, pbatch);
                        out_store(S, old, pend_full, pm0, pn0, pbatch, pslot);
                    }
                };
                static_for<PARTS>(step);
                pend = false;
            }
        }
        for (; kt < nk; ++kt) k_iteration(NoEp{});

        const bool full = nk == p.ktiles;
        T *slot = p.partials + ((int64_t)vb * 2 + (k_lo > 0 ? 0 : 1)) * ((int64_t)BM * BN);
        if constexpr (DEFER) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) old[i][j] = acc[i][j];
            pend = true;
            pend_full = full;
            pm0 = m0;
            pn0 = n0;
            pbatch = batch;
            pslot = slot;
        } else {
            auto whole = [&](auto S) __attribute__((always_inline)) {
                out_load(S, full, m0, n0, batch);
                out_store(S, acc, full, m0, n0, batch, slot);
            };
            static_for<PARTS>(whole);
        }
        it += nk;
    }
    if constexpr (DEFER) {
        if (pend) {
            auto whole = [&](auto S) __attribute__((always_inline)) {
                out_load(S, pend_full, pm0, pn0, pbatch);
                out_store(S, old, pend_full, pm0, pn0, pbatch, pslot);
            };
            static_for<PARTS>(whole);
        }
    }
}

// Completes the tiles whose K range was shared by several workgroups of gemm_kernel. Workgroup
// (b, part) (1 <= b < grid) looks at the boundary between main-kernel workgroups b - 1 and b; if
// that boundary falls inside a tile and is the FIRST such boundary of that tile, it adds the
// tile's slots in K order and applies the epilogue for one of kFixupParts equal shares of the
// values each thread owned in the main kernel.
constexpr int kFixupParts = 4;

template <typename T, int BM, int BN, int WM, int WN, typename M>
__global__ __launch_bounds__(WM *WN *kWave) void gemm_fixup_kernel(const GemmArgs<T> p) {
    using V = typename M::V;
    constexpr int MT = M::MT, EPV = M::EPV;
    constexpr int NT = WM * WN * kWave;
    constexpr int WTM = BM / WM, WTN = BN / WN;
    constexpr int TM = WTM / MT, TN = WTN / MT;
    constexpr int PER = TM * TN * M::ACC;   // values per thread and slot
    constexpr int PV = PER / kFixupParts;   // values this workgroup sums per thread
    constexpr int NV = PV / EPV;
    static_assert(PER % (kFixupParts * EPV) == 0 && M::ACC % EPV == 0, "slot share must be whole vectors");
    constexpr int64_t SLOT = (int64_t)BM * BN;
    const int grid = p.grid;
    const int64_t total = p.total_iters;
    const int b = (int)blockIdx.x + 1;
    const int64_t x = (int64_t)b * total / grid;  // first iteration of main-kernel workgroup b
    const int64_t tile = x / p.ktiles;
    const int64_t it0 = tile * p.ktiles;
    if (x == it0) return;  // boundary on a tile edge: nothing is split here
    auto owner_of = [&](int64_t i) { return (int)(((i + 1) * grid - 1) / total); };
    const int b_first = owner_of(it0), b_last = owner_of(it0 + p.ktiles - 1);
    if (b != b_first + 1) return;  // a later boundary of the same tile
    const int nseg = b_last - b_first + 1;

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int wm0 = (wave / WN) * WTM, wn0 = (wave % WN) * WTN, lrow = lane % MT;
    const int ev0 = (int)blockIdx.y * NV;  // first vector of this workgroup's share
    auto slot_of = [&](int ob) {
        const bool starts_inside = ((int64_t)ob * total / grid) > it0;
        return p.partials + ((int64_t)ob * 2 + (starts_inside ? 0 : 1)) * SLOT + ((int64_t)ev0 * NT + tid) * EPV;
    };
    // The first two contributions are fetched together (every split tile has at least two).
    V s0[NV], s1[NV];
    const T *src0 = slot_of(b_first), *src1 = slot_of(b_first + 1);
#pragma unroll
    for (int v = 0; v < NV; ++v) s0[v] = *reinterpret_cast<const V *>(src0 + (int64_t)v * NT * EPV);
#pragma unroll
    for (int v = 0; v < NV; ++v) s1[v] = *reinterpret_cast<const V *>(src1 + (int64_t)v * NT * EPV);
    T sum[PV];
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int q = 0; q < EPV; ++q) sum[v * EPV + q] = M::elem(s0[v], q) + M::elem(s1[v], q);
    for (int sgm = 2; sgm < nseg; ++sgm) {
        const T *src = slot_of(b_first + sgm);
#pragma unroll
        for (int v = 0; v < NV; ++v) s0[v] = *reinterpret_cast<const V *>(src + (int64_t)v * NT * EPV);
#pragma unroll
        for (int v = 0; v < NV; ++v)
#pragma unroll
            for (int q = 0; q < EPV; ++q) sum[v * EPV + q] = sum[v * EPV + q] + M::elem(s0[v], q);
    }

    const int64_t batch = tile / p.tiles_per_batch;
    int tile_m, tile_n;
    tile_of_id(tile - batch * p.tiles_per_batch, p.tiles_m, p.tiles_n, tile_m, tile_n, p.order);
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
    T *C = p.c + batch * p.stride_c;
    // Row maxima (GemmArgs::rowmax) of a split tile: with 16 x 16 accumulators this workgroup's share is exactly one row block
    // of each wavefront's part of the tile (TN accumulators, 4 values a lane of each), in the main kernel's lane layout, so
    // the same in-lane combination and fold apply.
    constexpr bool ROWMAX = std::is_same<T, float>::value && M::ACC == 4 && PV == M::ACC * TN;
    float seen[ROWMAX ? 4 : 1];
    if constexpr (ROWMAX) {
#pragma unroll
        for (int r = 0; r < 4; ++r) seen[r] = -__builtin_inff();
    }
    const bool has_bias = (p.epilogue & FTH_EPI_BIAS) != 0;
    const bool has_gelu = (p.epilogue & FTH_EPI_GELU) != 0;
    const bool has_gelu_tanh = (p.epilogue & FTH_EPI_GELU_TANH) != 0;
    const bool has_res = (p.epilogue & FTH_EPI_RESIDUAL) != 0;
#pragma unroll
    for (int u = 0; u < PV; ++u) {
        const int e = (int)blockIdx.y * PV + u;  // flat index (i * TN + j) * ACC + r of the main kernel
        const int r = e % M::ACC, j = (e / M::ACC) % TN, i = e / (M::ACC * TN);
        const int64_t col = n0 + wn0 + j * MT + lrow;
        const int64_t row = m0 + wm0 + i * MT + M::acc_row(r, lane);
        if (col < p.n && row < p.m) {
            T v = sum[u];
            if (p.use_alpha) v = p.alpha * v;
            if (has_bias) v = v + p.bias[col];
            if (has_gelu) v = M::gelu(v);
            if (has_gelu_tanh) v = M::gelu_tanh(v);
            if (has_res) v = v + p.residual[batch * p.stride_c + row * p.ldc + col];
            C[row * p.ldc + col] = v;
            if constexpr (ROWMAX) seen[r] = nan_max(seen[r], (float)v);
        }
    }
    if constexpr (ROWMAX) {
        if (p.rowmax != nullptr) {  // uniform: every lane takes part in the fold
            const int i = (int)blockIdx.y;  // the row block this share is
            const float mine = rowmax_fold(seen, lane);
            const int64_t row = m0 + wm0 + i * MT + M::acc_row(rowmax_elem_of_lane(lane), lane);
            const int64_t group = (n0 + wn0) / WTN;
            if ((lane & 15) < 4 && row < p.m) p.rowmax[group * p.m + row] = (T)mine;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Small problems (the 128-token transformer block: 17 to 67 MFLOP per product): one launch, no fix-up pass.
// A workgroup owns one 32 x 32 output tile and splits K across its NW wavefronts; each wavefront feeds the MFMA
// straight from global memory (a 128-bit load along k is four MFMA steps; the operands are small and L2-resident, and
// nothing in a workgroup would reuse an LDS copy), and the NW partial tiles are added through LDS in wavefront order,
// so the sum order is fixed by the shape. The large-tile kernels need a second launch to combine split tiles, which at
// this size costs as much as the product itself.
// ---------------------------------------------------------------------------------------------
template <int NW, bool TRANS_B>
__global__ __launch_bounds__(64 * NW) void gemm_small_kernel(const GemmArgs<float> p) {
    using M = Mfma<float>;
    __shared__ float part[NW][32][33];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lrow = lane & 31, g = lane >> 5;
    const int64_t batch = blockIdx.y;
    const int tile_m = (int)(blockIdx.x / p.tiles_n), tile_n = (int)(blockIdx.x % p.tiles_n);
    const int64_t m0 = (int64_t)tile_m * 32, n0 = (int64_t)tile_n * 32;
    const float *A = p.a + batch * p.stride_a;
    const float *B = p.b + batch * p.stride_b;
    // this wavefront's K range: whole groups of 8 (one 128-bit load per lane group), contiguous, in wavefront order
    const int groups = (int)(p.k / 8), per = (groups + NW - 1) / NW;
    const int g0 = wave * per, g1 = (g0 + per < groups) ? g0 + per : groups;
    int64_t ar = m0 + lrow, br = n0 + lrow;  // rows past the edge read the last valid row; they are never stored
    ar = ar < p.m ? ar : p.m - 1;
    br = br < p.n ? br : p.n - 1;
    const float *ap = A + ar * p.lda + 4 * g;
    const float *bp = TRANS_B ? B + br * p.ldb + 4 * g : B + (int64_t)(4 * g) * p.ldb + br;
    typename M::Acc acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll 8
    for (int t = g0; t < g1; ++t) {
        const float4 av = *reinterpret_cast<const float4 *>(ap + 8 * t);
        float4 bv;
        if (TRANS_B) {
            bv = *reinterpret_cast<const float4 *>(bp + 8 * t);
        } else {
            const float *bk = bp + (int64_t)(8 * t) * p.ldb;
            bv = make_float4(bk[0], bk[p.ldb], bk[2 * p.ldb], bk[3 * p.ldb]);
        }
        acc = M::mma(av.x, bv.x, acc);
        acc = M::mma(av.y, bv.y, acc);
        acc = M::mma(av.z, bv.z, acc);
        acc = M::mma(av.w, bv.w, acc);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) part[wave][M::acc_row(r, lane)][lrow] = acc[r];
    __syncthreads();
    const bool has_bias = (p.epilogue & FTH_EPI_BIAS) != 0, has_gelu = (p.epilogue & FTH_EPI_GELU) != 0;
    const bool has_gelu_tanh = (p.epilogue & FTH_EPI_GELU_TANH) != 0, has_res = (p.epilogue & FTH_EPI_RESIDUAL) != 0;
    float *C = p.c + batch * p.stride_c;
#pragma unroll
    for (int e = tid; e < 1024; e += 64 * NW) {
        const int r = e >> 5, c = e & 31;
        const int64_t row = m0 + r, col = n0 + c;
        if (row < p.m && col < p.n) {
            float v = part[0][r][c];
#pragma unroll
            for (int w = 1; w < NW; ++w) v += part[w][r][c];
            if (p.use_alpha) v = p.alpha * v;
            if (has_bias) v = v + p.bias[col];
            if (has_gelu) v = M::gelu(v);
            if (has_gelu_tanh) v = M::gelu_tanh(v);
            if (has_res) v = v + p.residual[batch * p.stride_c + row * p.ldc + col];
            C[row * p.ldc + col] = v;
        }
    }
}

// The same for long reductions (k >= 512) with 16 x 16 output tiles (v_mfma_f32_16x16x4_f32): four times the workgroups, and
// a wavefront load covers 64 contiguous bytes of each of 16 rows instead of 32 bytes of each of 32. With 32 x 32 tiles a
// [128, 256] x k = 1024 product kept only 32 compute units busy and each spent its time moving 256 KiB of operands through its
// one vector memory pipe.
template <int NW, bool TRANS_B>
__global__ __launch_bounds__(64 * NW) void gemm_small16_kernel(const GemmArgs<float> p) {
    using M = Mfma<float>;
    typedef float Acc4 __attribute__((ext_vector_type(4)));
    __shared__ float part[NW][16][17];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lrow = lane & 15, g = lane >> 4;
    const int64_t batch = blockIdx.y;
    const int tile_m = (int)(blockIdx.x / p.tiles_n), tile_n = (int)(blockIdx.x % p.tiles_n);
    const int64_t m0 = (int64_t)tile_m * 16, n0 = (int64_t)tile_n * 16;
    const float *A = p.a + batch * p.stride_a;
    const float *B = p.b + batch * p.stride_b;
    // this wavefront's K range: whole groups of 16 (one 128-bit load per lane group), contiguous, in wavefront order
    const int groups = (int)(p.k / 16), per = (groups + NW - 1) / NW;
    const int g0 = wave * per, g1 = (g0 + per < groups) ? g0 + per : groups;
    int64_t ar = m0 + lrow, br = n0 + lrow;  // rows past the edge read the last valid row; they are never stored
    ar = ar < p.m ? ar : p.m - 1;
    br = br < p.n ? br : p.n - 1;
    const float *ap = A + ar * p.lda + 4 * g;
    const float *bp = TRANS_B ? B + br * p.ldb + 4 * g : B + (int64_t)(4 * g) * p.ldb + br;
    Acc4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
    for (int t = g0; t < g1; ++t) {
        const float4 av = *reinterpret_cast<const float4 *>(ap + 16 * t);
        float4 bv;
        if (TRANS_B) {
            bv = *reinterpret_cast<const float4 *>(bp + 16 * t);
        } else {
            const float *bk = bp + (int64_t)(16 * t) * p.ldb;
            bv = make_float4(bk[0], bk[p.ldb], bk[2 * p.ldb], bk[3 * p.ldb]);
        }
        // step i contracts k = 16 t + 4 g + i over the four lane groups
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av.x, bv.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av.y, bv.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av.z, bv.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av.w, bv.w, acc, 0, 0, 0);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) part[wave][4 * g + r][lrow] = acc[r];  // accumulator element r: row 4 (lane / 16) + r, column lane % 16
    __syncthreads();
    const bool has_bias = (p.epilogue & FTH_EPI_BIAS) != 0, has_gelu = (p.epilogue & FTH_EPI_GELU) != 0;
    const bool has_gelu_tanh = (p.epilogue & FTH_EPI_GELU_TANH) != 0, has_res = (p.epilogue & FTH_EPI_RESIDUAL) != 0;
    float *C = p.c + batch * p.stride_c;
    if (tid < 256) {
        const int r = tid >> 4, c = tid & 15;
        const int64_t row = m0 + r, col = n0 + c;
        if (row < p.m && col < p.n) {
            float v = part[0][r][c];
#pragma unroll
            for (int w = 1; w < NW; ++w) v += part[w][r][c];
            if (p.use_alpha) v = p.alpha * v;
            if (has_bias) v = v + p.bias[col];
            if (has_gelu) v = M::gelu(v);
            if (has_gelu_tanh) v = M::gelu_tanh(v);
            if (has_res) v = v + p.residual[batch * p.stride_c + row * p.ldc + col];
            C[row * p.ldc + col] = v;
        }
    }
}

// True (and the kernel launched) when the problem is one of the small ones this kernel is for.
template <bool TRANS_B> bool launch_small(GemmArgs<float> &p, int64_t batch, bool vec_a, bool vec_b, hipStream_t st, int32_t *rc) {
    static const bool off = [] {
        const char *e = std::getenv("FT_HIP_GEMM_SMALL");  // tuning knob: 0 sends small problems to the large-tile kernels
        return e && std::atoi(e) == 0;
    }();
    const int64_t tiles = fth::ceil_div(p.m, 32) * fth::ceil_div(p.n, 32);
    double flop = 2.0 * (double)p.m * (double)p.n * (double)p.k * (double)batch;
    if (off || !vec_a || (TRANS_B && !vec_b) || p.k % 8 != 0 || p.k < 64 || flop > 4.0e8 || tiles > 2147483647LL || batch > 65535) return false;
    p.tiles_m = (int)fth::ceil_div(p.m, 32);
    p.tiles_n = (int)fth::ceil_div(p.n, 32);
    const dim3 grid((unsigned)tiles, (unsigned)batch);
    const int64_t tiles16 = fth::ceil_div(p.m, 16) * fth::ceil_div(p.n, 16);
    if (p.k < 512) {
        gemm_small_kernel<4, TRANS_B><<<grid, dim3(256), 0, st>>>(p);
    } else if (p.k % 16 == 0 && tiles16 * batch <= 4096) {  // long reduction, few tiles: 16 x 16 tiles on four times the compute units
        p.tiles_m = (int)fth::ceil_div(p.m, 16);
        p.tiles_n = (int)fth::ceil_div(p.n, 16);
        gemm_small16_kernel<8, TRANS_B><<<dim3((unsigned)tiles16, (unsigned)batch), dim3(512), 0, st>>>(p);
    } else if (p.k <= 512) {
        gemm_small_kernel<4, TRANS_B><<<grid, dim3(256), 0, st>>>(p);
    } else {
        gemm_small_kernel<8, TRANS_B><<<grid, dim3(512), 0, st>>>(p);
    }
    hipError_t e = hipGetLastError();
    *rc = e == hipSuccess ? FTH_OK : fth::hip_fail(e, "gemm_small");
    return true;
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
    if (p.epilogue & FTH_EPI_GELU_TANH) v = M::gelu_tanh(v);
    if (p.epilogue & FTH_EPI_RESIDUAL) v = v + p.residual[batch * p.stride_c + row * p.ldc + col];
    p.c[batch * p.stride_c + row * p.ldc + col] = v;
}

// Workspace of split tiles, one per stream (two GEMMs on different streams may overlap).
struct StreamWorkspace {
    void *partials = nullptr;
    size_t partial_bytes = 0;
};
// slot 0: split-tile accumulators; slot 1: transposed copy of a [k, m] A operand.
//
// A block that a larger request outgrows is retired, never handed back to the shared pool: kernels
// queued on the stream may still be using it, the pool serves every stream and thread (so "ordered
// on the same stream" would not protect the next owner), and a captured HIP graph keeps the address
// it was recorded with for as long as its executable lives. Requests up to 4 GiB grow geometrically,
// so the retired blocks of a (stream, slot) add up to less than its current one; only a single
// request beyond 4 GiB (a transposed operand of more than 2^30 floats) retires its predecessor without
// that bound. The totals are reported by fth_device_workspace_info.
struct WorkspaceTable {
    std::mutex mu;
    std::map<std::pair<hipStream_t, int>, StreamWorkspace> table;
    std::vector<void *> retired;
    uint64_t live_bytes = 0, retired_bytes = 0;
};
WorkspaceTable &workspace_table() {
    static WorkspaceTable *t = new WorkspaceTable();  // never destroyed: streams outlive static destructors
    return *t;
}
int32_t get_workspace(hipStream_t st, size_t partial_bytes, void **partials, int slot = 0) {
    WorkspaceTable &t = workspace_table();
    std::lock_guard<std::mutex> lock(t.mu);
    StreamWorkspace &w = t.table[std::make_pair(st, slot)];
    if (w.partial_bytes < partial_bytes) {
        size_t want = partial_bytes;
        if (w.partial_bytes && want < 2 * w.partial_bytes && w.partial_bytes <= ((size_t)1 << 31)) want = 2 * w.partial_bytes;
        void *fresh = nullptr;
        if (int32_t rc = fth::pool_alloc(&fresh, want)) {
            if (want == partial_bytes) return rc;
            want = partial_bytes;  // the doubled block did not fit: take exactly what is needed
            if (int32_t rc2 = fth::pool_alloc(&fresh, want)) return rc2;
        }
        if (w.partials) {
            t.retired.push_back(w.partials);
            t.retired_bytes += w.partial_bytes;
            t.live_bytes -= w.partial_bytes;
        }
        w.partials = fresh;
        w.partial_bytes = want;
        t.live_bytes += want;
    }
    *partials = w.partials;
    return FTH_OK;
}

constexpr int kMinItersPerBlock = 4;  // never cut the iteration space finer than this many K-tiles

// Launches a persistent main kernel over the stream-K schedule, then the fix-up kernel if any
// tile is split. `blocks_per_cu` caches the kernel's occupancy (one static per kernel).
template <typename T, int BM, int BN, int WM, int WN, typename MM, typename Kern>
int32_t launch_persistent(Kern kern, size_t smem, int BK, int &blocks_per_cu, GemmArgs<T> &p, int64_t batch, hipStream_t st) {
    constexpr int NT = WM * WN * kWave;
    if (blocks_per_cu == 0) {  // benign race: both calls are idempotent
        FTH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        int nb = 0;
        FTH_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, kern, NT, smem));
        blocks_per_cu = nb > 0 ? nb : 1;
    }
    const int64_t tm = fth::ceil_div(p.m, BM), tn = fth::ceil_div(p.n, BN);
    const int64_t ktiles = fth::ceil_div(p.k, BK);
    FTH_ARG(tm <= 2147483647LL && tn <= 2147483647LL && ktiles <= 2147483647LL, "gemm: extent too large");
    int64_t tiles, total;
    if (__builtin_mul_overflow(tm, tn, &tiles) || __builtin_mul_overflow(tiles, batch, &total) || total > 2147483647LL ||
        __builtin_mul_overflow(total, ktiles, &total) || total > (int64_t)1 << 46)
        return fth::set_error(FTH_ERR_SIZE_OVERFLOW, "gemm: too many tiles (%lld x %lld x batch %lld)", (long long)tm, (long long)tn,
                              (long long)batch);
    const int cus = fth::compute_units() > 0 ? fth::compute_units() : 256;
    int64_t grid = (int64_t)cus * blocks_per_cu;
    const int64_t cap = total / kMinItersPerBlock > 0 ? total / kMinItersPerBlock : 1;
    if (grid > cap) grid = cap;
    {
        static const int forced_grid = [] {
            const char *e = std::getenv("FT_HIP_GEMM_GRID");  // tuning knob: workgroups of the persistent kernels
            return e ? std::atoi(e) : 0;
        }();
        if (forced_grid > 0 && forced_grid <= grid) grid = forced_grid;
    }
    p.tiles_m = (int)tm;
    p.tiles_n = (int)tn;
    p.ktiles = (int)ktiles;
    p.tiles_per_batch = tm * tn;
    p.total_iters = total;
    p.grid = (int)grid;
    {
        static const int forced_order = [] {
            const char *e = std::getenv("FT_HIP_GEMM_TILE_ORDER");  // tuning knob: 0 / 1 force the tile order of tile_of_id
            return e ? std::atoi(e) : -1;
        }();
        p.order = forced_order == 0 || forced_order == 1 ? forced_order : (tn > tm ? 1 : 0);  // wide outputs walk along their rows
    }
    // A tile is split when a workgroup boundary b * total / grid is not a multiple of ktiles.
    bool any_split = false;
    if (grid > 1) {
        const int64_t per = total / grid;
        any_split = !(total % grid == 0 && per % ktiles == 0);
    }
    void *partials = nullptr;
    if (any_split)
        if (int32_t rc = get_workspace(st, (size_t)grid * 2 * BM * BN * sizeof(T), &partials)) return rc;
    p.partials = static_cast<T *>(partials);
    kern<<<dim3((unsigned)grid), dim3(NT), smem, st>>>(p);
    FTH_CHECK_LAUNCH("gemm");
    if (any_split) {
        gemm_fixup_kernel<T, BM, BN, WM, WN, MM><<<dim3((unsigned)(grid - 1), kFixupParts), dim3(NT), 0, st>>>(p);
        FTH_CHECK_LAUNCH("gemm_fixup");
    }
    return FTH_OK;
}

template <typename T, int BM, int BN, int BK, int WM, int WN, int MINW, bool TRANS_B, bool VEC, bool VECB>
int32_t launch_config(GemmArgs<T> &p, int64_t batch, hipStream_t st) {
    constexpr int S = BK + Mfma<T>::EPV;
    constexpr size_t smem = (size_t)2 * (BM + BN) * S * sizeof(T);
    static int blocks_per_cu = 0;
    return launch_persistent<T, BM, BN, WM, WN, Mfma<T>>(gemm_kernel<T, BM, BN, BK, WM, WN, MINW, TRANS_B, VEC, VECB>, smem, BK, blocks_per_cu, p,
                                                 batch, st);
}

template <typename T, int BM, int BN, int WM, int WN, int MINW, bool TRANS_A, bool TRANS_B, int EPI>
int32_t launch_direct_epi(GemmArgs<T> &p, int64_t batch, hipStream_t st) {
    constexpr int BK = 128 / (int)sizeof(T);
    constexpr size_t smem = (size_t)2 * (BM + BN) * BK * sizeof(T);
    static int blocks_per_cu = 0;
    return launch_persistent<T, BM, BN, WM, WN, typename DirectMfma<T, BM, BN, TRANS_A, TRANS_B, EPI>::type>(
        gemm_direct_kernel<T, BM, BN, WM, WN, MINW, TRANS_A, TRANS_B, EPI>, smem, BK, blocks_per_cu, p,
                                                 batch, st);
}

// SPECIALIZE: pick a kernel with the epilogue flags compiled in for the combinations the
// transformer block uses (none, bias, bias+GELU in either form, bias+residual; alpha = 1).
template <typename T, int BM, int BN, int WM, int WN, int MINW, bool TRANS_B, bool SPECIALIZE>
int32_t launch_direct(GemmArgs<T> &p, int64_t batch, hipStream_t st) {
    if constexpr (SPECIALIZE) {
        if (!p.use_alpha) {
            switch (p.epilogue) {
                case 0: return launch_direct_epi<T, BM, BN, WM, WN, MINW, false, TRANS_B, 0>(p, batch, st);
                case FTH_EPI_BIAS: return launch_direct_epi<T, BM, BN, WM, WN, MINW, false, TRANS_B, FTH_EPI_BIAS>(p, batch, st);
                case FTH_EPI_BIAS | FTH_EPI_GELU:
                    return launch_direct_epi<T, BM, BN, WM, WN, MINW, false, TRANS_B, FTH_EPI_BIAS | FTH_EPI_GELU>(p, batch, st);
                case FTH_EPI_BIAS | FTH_EPI_GELU_TANH:
                    return launch_direct_epi<T, BM, BN, WM, WN, MINW, false, TRANS_B, FTH_EPI_BIAS | FTH_EPI_GELU_TANH>(p, batch, st);
                case FTH_EPI_BIAS | FTH_EPI_RESIDUAL:
                    return launch_direct_epi<T, BM, BN, WM, WN, MINW, false, TRANS_B, FTH_EPI_BIAS | FTH_EPI_RESIDUAL>(p, batch, st);
                default: break;
            }
        }
    }
    return launch_direct_epi<T, BM, BN, WM, WN, MINW, false, TRANS_B, -1>(p, batch, st);
}

// 128x128 tiles when there is one per CU, or when K is long enough that the stream-K split still
// leaves every resident workgroup a run of at least 16 K-tiles (few tiles, deep K: weight gradients).
inline bool use_big_tiles(int64_t big_tiles, int64_t k, int cus) {
    return big_tiles >= cus || big_tiles * fth::ceil_div(k, 32) >= (int64_t)cus * 2 * 16;
}

// Tile configurations. The choice depends on the shape only (never on timing), so a given problem
// always runs the same kernel and reproduces its bits.
enum class Tile { Big, Wide, Small, Tall };

inline int forced_tile() {
    static const int v = [] {
        const char *e = std::getenv("FT_HIP_GEMM_TILE");  // tuning knob: 0 = 128x128, 1 = 256x128, 2 = 64x64, 3 = 128x64, 4 = 128x96 (3, 4: direct fp32 only)
        return e ? std::atoi(e) : -1;
    }();
    return v;
}

template <typename T, bool TRANS_B, bool VEC, bool VECB>
int32_t launch_shape(GemmArgs<T> &p, int64_t batch, hipStream_t st) {
    // Large problems: 128x128 tiles (2x2 wavefronts of 64x64). Problems too small to give every
    // CU a large tile: 64x64 tiles (2x2 wavefronts of 32x32).
    const int64_t big_tiles = fth::ceil_div(p.m, 128) * fth::ceil_div(p.n, 128) * batch;
    const int cus = fth::compute_units() > 0 ? fth::compute_units() : 256;
    Tile t = use_big_tiles(big_tiles, p.k, cus) ? Tile::Big : Tile::Small;
    const int f = forced_tile();
    if (f == 0) t = Tile::Big;
    if (f == 1) t = Tile::Wide;
    if (f == 2) t = Tile::Small;
    if constexpr (VEC && (TRANS_B || VECB)) {
        // 16-byte aligned operand rows: direct-to-LDS kernel when K is a whole number of 128-byte
        // K-tiles and a tile's lane offsets fit 32 bits.
        constexpr int64_t DBK = 128 / (int64_t)sizeof(T);
        static const bool direct_off = [] {
            const char *e = std::getenv("FT_HIP_GEMM_DIRECT");  // tuning knob: 0 disables the direct-to-LDS kernels
            return e && std::atoi(e) == 0;
        }();
        const int64_t lim = ((int64_t)1 << 32) / (128 * (int64_t)sizeof(T)) - 128;  // a tile's lane byte offsets fit 32 bits
        if (!direct_off && t != Tile::Wide && p.k % DBK == 0 && p.lda <= lim && p.ldb <= lim && p.ldc <= lim) {
            constexpr int MINW_BIG = 2;
            if constexpr (std::is_same<T, float>::value) {
                {
                    // 128x96 tiles (4x1 wavefronts of 32x96) when they hand every resident workgroup (two per compute
                    // unit) a whole number of whole tiles and 128x128 tiles do not: no tile is split over K, no fix-up
                    // pass. All GPT-2 widths are multiples of 96 (768 = 8 x 96): QKV 0.77 -> 0.82, O-proj 0.75 -> 0.78,
                    // FC2 0.82 -> 0.83 of the matrix peak; where 128x128 tiles already divide evenly (FC1) they stay
                    // (their main loop is 1-2 % faster). With B stored [k, n] the same holds for the input gradient of
                    // a linear layer (dy . W at FC2's shape).
                    const int64_t slots = (int64_t)cus * 2;
                    const int64_t tiles96 = fth::ceil_div(p.m, 128) * (p.n / 96) * batch;
                    const bool n96 = f < 0 && t == Tile::Big && p.n % 96 == 0 && tiles96 % slots == 0 && big_tiles % slots != 0;
                    if (n96 || f == 4) return launch_direct<T, 128, 96, 4, 1, 2, TRANS_B, true>(p, batch, st);
                }
                // Fewer 128x128 tiles than resident workgroups would split every tile over K; 128x64
                // tiles (three workgroups per CU) give each workgroup whole tiles instead. Their main
                // loop is about 8 % slower, which costs more than the fix-up pass (about 25 us) once
                // the problem exceeds some 30 GFLOP.
                const int64_t tall_tiles = fth::ceil_div(p.m, 128) * fth::ceil_div(p.n, 64) * batch;
                const double flop = 2.0 * (double)p.m * (double)p.n * (double)p.k * (double)batch;
                if (f < 0 && t == Tile::Big && big_tiles < 2 * (int64_t)cus && tall_tiles >= 2 * (int64_t)cus && flop < 30e9) t = Tile::Tall;
                if (f == 3) t = Tile::Tall;
                if (t == Tile::Tall) return launch_direct<T, 128, 64, 2, 2, 3, TRANS_B, true>(p, batch, st);
            }
            if (t == Tile::Big) return launch_direct<T, 128, 128, 2, 2, MINW_BIG, TRANS_B, std::is_same<T, float>::value>(p, batch, st);
            return launch_direct<T, 64, 64, 2, 2, 2, TRANS_B, false>(p, batch, st);
        }
    }
    if constexpr (std::is_same<T, float>::value) {
        switch (t) {
            case Tile::Big: return launch_config<T, 128, 128, FTH_F32_BK, 2, 2, FTH_F32_MINW, TRANS_B, VEC, VECB>(p, batch, st);
            case Tile::Wide: return launch_config<T, 256, 128, 16, 2, 2, 2, TRANS_B, VEC, VECB>(p, batch, st);
            default: return launch_config<T, 64, 64, 32, 2, 2, 1, TRANS_B, VEC, VECB>(p, batch, st);
        }
    } else {
        switch (t) {
            case Tile::Big:
            case Tile::Wide: return launch_config<T, 128, 128, 16, 2, 2, 1, TRANS_B, VEC, VECB>(p, batch, st);
            default: return launch_config<T, 64, 64, 16, 2, 2, 1, TRANS_B, VEC, VECB>(p, batch, st);
        }
    }
}

// dst[b][i][j] = src[b][j][i]: src is [rows, cols] with pitch ld_src, dst is [cols, rows] contiguous.
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(const T *src, T *dst, int64_t rows, int64_t cols, int64_t ld_src,
                                                        int64_t stride_src, int64_t stride_dst) {
    __shared__ T tile[32][33];
    const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;  // 32 x 8
    const int64_t r0 = (int64_t)blockIdx.y * 32, c0 = (int64_t)blockIdx.x * 32;
    src += (int64_t)blockIdx.z * stride_src;
    dst += (int64_t)blockIdx.z * stride_dst;
#pragma unroll
    for (int i = 0; i < 32; i += 8) {
        const int64_t r = r0 + ty + i, c = c0 + tx;
        tile[ty + i][tx] = (r < rows && c < cols) ? src[r * ld_src + c] : T(0);
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 32; i += 8) {
        const int64_t c = c0 + ty + i, r = r0 + tx;
        if (c < cols && r < rows) dst[c * rows + r] = tile[tx][ty + i];
    }
}

// A stored [k, m]: gemm::sgemm_tb / dgemm_tb (crates/ft-kernel-cpu/src/lib.rs:1484-1524, 262-345).
// With 16-byte aligned rows of both operands and K a whole number of K-tiles the direct-to-LDS
// kernel reads A as stored; other shapes go through a transposed copy and the [m, k] path.
template <typename T> int32_t launch_trans_a(GemmArgs<T> &p, const fth_gemm_desc *d, hipStream_t st);

template <typename T>
int32_t gemm_entry(const fth_gemm_desc *d, T alpha, const T *a, const T *b, T *c, const T *bias, const T *residual,
                   fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(d != nullptr, "gemm: desc is NULL");
    FTH_ARG(d->m >= 0 && d->n >= 0 && d->k >= 0 && d->batch >= 0, "gemm: negative extent");
    if (d->m == 0 || d->n == 0 || d->batch == 0) return FTH_OK;  // crates/ft-kernel-cpu/src/lib.rs:1311-1313
    FTH_ARG(c != nullptr, "gemm: C is NULL");
    FTH_ARG(d->k == 0 || (a && b), "gemm: NULL operand");
    FTH_ARG(d->lda >= (d->trans_a ? d->m : d->k) && d->ldc >= d->n && d->ldb >= (d->trans_b ? d->k : d->n),
            "gemm: row pitch smaller than the row (lda %lld ldb %lld ldc %lld)", (long long)d->lda, (long long)d->ldb,
            (long long)d->ldc);
    FTH_ARG(!(d->trans_a && d->trans_b), "gemm: trans_a together with trans_b is not supported");
    FTH_ARG(!(d->epilogue & FTH_EPI_BIAS) || bias, "gemm: bias epilogue without a bias pointer");
    FTH_ARG(!(d->epilogue & FTH_EPI_RESIDUAL) || residual, "gemm: residual epilogue without a residual pointer");
    FTH_ARG((d->epilogue & ~(FTH_EPI_BIAS | FTH_EPI_GELU | FTH_EPI_RESIDUAL | FTH_EPI_GELU_TANH)) == 0, "gemm: unknown epilogue bits");
    FTH_ARG((d->epilogue & (FTH_EPI_GELU | FTH_EPI_GELU_TANH)) != (FTH_EPI_GELU | FTH_EPI_GELU_TANH), "gemm: both GELU forms requested");
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
    if (d->trans_a) return launch_trans_a<T>(p, d, st);
    constexpr int EPV = Mfma<T>::EPV;
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    // 128-bit global loads along k need 16-byte aligned rows in every batch.
    bool vec = d->k % EPV == 0 && d->lda % EPV == 0 && al(a) && d->stride_a % EPV == 0;
    if (d->trans_b) vec = vec && d->ldb % EPV == 0 && al(b) && d->stride_b % EPV == 0;
    if constexpr (std::is_same<T, float>::value) {
        int32_t rc = FTH_OK;
        const bool vec_bt = d->ldb % EPV == 0 && al(b) && d->stride_b % EPV == 0;
        if (d->trans_b ? launch_small<true>(p, d->batch, vec, vec_bt, st, &rc) : launch_small<false>(p, d->batch, vec, true, st, &rc)) return rc;
    }
    if (d->trans_b) {
        return vec ? launch_shape<T, true, true, false>(p, d->batch, st) : launch_shape<T, true, false, false>(p, d->batch, st);
    }
    // [k, n] B: 128-bit loads along n need n, ldb and the base to be vector multiples (and k, so
    // that a register block never straddles the k edge).
    const bool vecb = d->n % EPV == 0 && d->k % EPV == 0 && d->ldb % EPV == 0 && al(b) && d->stride_b % EPV == 0;
    if (vec) return vecb ? launch_shape<T, false, true, true>(p, d->batch, st) : launch_shape<T, false, true, false>(p, d->batch, st);
    return vecb ? launch_shape<T, false, false, true>(p, d->batch, st) : launch_shape<T, false, false, false>(p, d->batch, st);
}

// C = A . B^T (A [m, k], B [n, k], both row-major and contiguous) on 128 x 128 tiles with the row maxima of every 64-column
// group as a by-product (GemmArgs::rowmax). Returns false, with nothing launched, where the direct-to-LDS kernel or the
// large tiles do not apply.
bool launch_nt_rowmax(int64_t m, int64_t n, int64_t k, const float *a, const float *b, float *c, float *rowmax, hipStream_t st, int32_t *rc) {
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    const int64_t lim = ((int64_t)1 << 32) / (128 * (int64_t)sizeof(float)) - 128;
    const int cus = fth::compute_units() > 0 ? fth::compute_units() : 256;
    const int64_t big_tiles = fth::ceil_div(m, 128) * fth::ceil_div(n, 128);
    static const bool direct_off = [] {
        const char *e = std::getenv("FT_HIP_GEMM_DIRECT");
        return e && std::atoi(e) == 0;
    }();
    if (direct_off || m <= 0 || n <= 0 || k <= 0 || k % 32 != 0 || !al(a) || !al(b) || k > lim || n > lim || big_tiles < cus || forced_tile() > 0)
        return false;
    GemmArgs<float> p;
    p.a = a; p.b = b; p.c = c; p.bias = nullptr; p.residual = nullptr;
    p.m = m; p.n = n; p.k = k;
    p.lda = k; p.ldb = k; p.ldc = n;
    p.stride_a = m * k; p.stride_b = n * k; p.stride_c = m * n;
    p.alpha = 1.f;
    p.use_alpha = 0;
    p.epilogue = 0;
    p.tiles_m = p.tiles_n = 0;
    p.rowmax = rowmax;
    *rc = launch_direct_epi<float, 128, 128, 2, 2, 2, false, true, kEpiRowMax>(p, 1, st);
    return true;
}

template <typename T> int32_t launch_trans_a(GemmArgs<T> &p, const fth_gemm_desc *d, hipStream_t st) {
    constexpr int EPV = Mfma<T>::EPV;
    constexpr int64_t DBK = 128 / (int64_t)sizeof(T);
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    const int64_t lim = ((int64_t)1 << 32) / (128 * (int64_t)sizeof(T)) - 128;  // a tile's lane byte offsets fit 32 bits
    const bool direct = d->m % EPV == 0 && d->n % EPV == 0 && d->k % DBK == 0 && d->lda % EPV == 0 && d->ldb % EPV == 0 &&
                        d->stride_a % EPV == 0 && d->stride_b % EPV == 0 && al(p.a) && al(p.b) && d->lda <= lim && d->ldb <= lim &&
                        d->ldc <= lim;
    if (direct) {
        const int64_t big_tiles = fth::ceil_div(p.m, 128) * fth::ceil_div(p.n, 128) * d->batch;
        const int cus = fth::compute_units() > 0 ? fth::compute_units() : 256;
        if (use_big_tiles(big_tiles, p.k, cus)) return launch_direct_epi<T, 128, 128, 2, 2, 2, true, false, -1>(p, d->batch, st);
        return launch_direct_epi<T, 64, 64, 2, 2, 2, true, false, -1>(p, d->batch, st);
    }
    // Transposed copy A^T [batch][m][k], then the ordinary [m, k] path.
    size_t elems;
    if (__builtin_mul_overflow((size_t)d->m, (size_t)d->k, &elems) || __builtin_mul_overflow(elems, (size_t)d->batch, &elems) ||
        elems > ((size_t)1 << 40))
        return fth::set_error(FTH_ERR_SIZE_OVERFLOW, "gemm: transposed copy of A too large");
    void *ws = nullptr;
    if (int32_t rc = get_workspace(st, elems * sizeof(T), &ws, 1)) return rc;
    FTH_ARG(d->batch <= 65535 && fth::ceil_div(d->k, 32) <= 65535, "gemm: transposed copy grid too large");
    transpose_kernel<T><<<dim3((unsigned)fth::ceil_div(d->m, 32), (unsigned)fth::ceil_div(d->k, 32), (unsigned)d->batch), dim3(256), 0, st>>>(
        p.a, static_cast<T *>(ws), d->k, d->m, d->lda, d->stride_a, d->m * d->k);
    FTH_CHECK_LAUNCH("gemm_transpose_a");
    fth_gemm_desc d2 = *d;
    d2.trans_a = 0;
    d2.lda = d->k;
    d2.stride_a = d->m * d->k;
    return gemm_entry<T>(&d2, p.alpha, static_cast<const T *>(ws), p.b, p.c, p.bias, p.residual, reinterpret_cast<fth_stream>(st));
}

}  // namespace

namespace fth {
int64_t gemm_rowmax_groups(int64_t n) { return fth::ceil_div(n, 128) * 2; }
bool gemm_f32_nt_rowmax(int64_t m, int64_t n, int64_t k, const float *a, const float *b, float *c, float *rowmax, hipStream_t st,
                        int32_t *rc) {
    return launch_nt_rowmax(m, n, k, a, b, c, rowmax, st, rc);
}
}  // namespace fth

extern "C" {

int64_t fth_dev_linear_argmax_workspace_floats(int64_t rows, int64_t out_features) {
    if (rows <= 0 || out_features <= 0) return 0;
    return rows * fth::gemm_rowmax_groups(out_features);
}

int32_t fth_dev_linear_argmax_f32(const float *x, const float *w, int64_t rows, int64_t out_features, int64_t in_features,
                                  float *logits, float *argmax, float *workspace, int64_t workspace_floats, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(rows >= 0 && out_features >= 0 && in_features >= 0, "linear_argmax: negative extent");
    if (rows == 0) return FTH_OK;
    FTH_ARG(out_features > 0, "linear_argmax: argmax over an empty dimension");
    FTH_ARG(x && w && logits && argmax, "linear_argmax: NULL operand");
    hipStream_t st = fth::resolve_stream(s);
    static const bool fused_off = [] {
        const char *e = std::getenv("FT_HIP_LINEAR_ARGMAX_FUSED");  // tuning knob: 0 = always the two separate kernels
        return e && std::atoi(e) == 0;
    }();
    if (!fused_off && workspace && workspace_floats >= fth_dev_linear_argmax_workspace_floats(rows, out_features)) {
        int32_t rc = FTH_OK;
        if (fth::gemm_f32_nt_rowmax(rows, out_features, in_features, x, w, logits, workspace, st, &rc)) {
            if (rc) return rc;
            return fth::argmax_from_group_max(logits, rows, out_features, workspace, fth::gemm_rowmax_groups(out_features), argmax, st);
        }
    }
    fth_gemm_desc gd{};
    gd.m = rows; gd.n = out_features; gd.k = in_features; gd.batch = 1;
    gd.lda = in_features; gd.ldb = in_features; gd.ldc = out_features;
    gd.trans_b = 1;
    gd.epilogue = FTH_EPI_NONE;
    if (int32_t rc = fth_dev_gemm_f32(&gd, 1.f, x, w, logits, nullptr, nullptr, s)) return rc;
    return fth_dev_argmax_f32(logits, rows, out_features, 1, argmax, s);
}

int32_t fth_device_workspace_info(uint64_t *live_bytes, uint64_t *retired_bytes) {
    WorkspaceTable &t = workspace_table();
    std::lock_guard<std::mutex> lock(t.mu);
    if (live_bytes) *live_bytes = t.live_bytes;
    if (retired_bytes) *retired_bytes = t.retired_bytes;
    return FTH_OK;
}

int32_t fth_dev_gemm_f32(const fth_gemm_desc *d, float alpha, const float *a, const float *b, float *c,
                         const float *bias, const float *residual, fth_stream s) {
    return gemm_entry<float>(d, alpha, a, b, c, bias, residual, s);
}

int32_t fth_dev_gemm_f64(const fth_gemm_desc *d, double alpha, const double *a, const double *b, double *c,
                         const double *bias, const double *residual, fth_stream s) {
    return gemm_entry<double>(d, alpha, a, b, c, bias, residual, s);
}

}  // extern "C"
