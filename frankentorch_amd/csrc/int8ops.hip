// Int8 dynamic-quantised linear layer on the gfx950 integer matrix cores.
//
// replaces quantize_rows_i8 (crates/ft-kernel-cpu/src/lib.rs:37879-37905), quantize_per_output_channel_i8
// (:37836-37868) and linear_int8_dynamic_f32 (:37966-38060):
//     y[s, o] = (float)(sum_i xq[s, i] * wq[o, i]) * a_scale[s] * w_scale[o] (+ bias[o])
// with xq = per-row symmetric int8 of x (scale = max|row| / 127, or 1 for an all-zero row;
// round-ties-even, clamp to +-127). The products accumulate in int32, so the result does not depend on
// the order of the sum and every output equals the reference's bit for bit; the three float operations
// of the dequantisation are kept apart (this file is built without contraction).
//
// Product kernel: v_mfma_i32_32x32x32_i8, 256 x 256 output tile per workgroup (2 x 2 wavefronts of 128 x 128;
// 128 x 128 tiles for problems with few tiles), K in steps of 64 bytes through a ring of four LDS stages filled by global_load_lds_dwordx4 (a
// stage of this kernel is only 256 MFMA cycles per wavefront, far less than a memory round trip, so three
// stages are kept in flight). Both
// operands are k-contiguous ([m, k] activations, [n, k] weights), so a lane's fragment is 16 consecutive
// bytes of one row. Rows are 64 bytes in LDS; 16-byte slot q of row r is stored at q ^ ((r >> 2) & 3),
// which spreads any 16 consecutive rows of one slot over all 64 banks. Rows past m / n are clamped to the
// last valid row on the load side and never stored. Shapes whose K is not a multiple of 64 or whose
// operands are not 16-byte aligned take a plain one-thread-per-output kernel.

#include <cstdlib>

#include <type_traits>

#include "common.hpp"

namespace {

constexpr int kWave = 64;
using V4i = int __attribute__((ext_vector_type(4)));
using V16i = int __attribute__((ext_vector_type(16)));

// ---- quantisation: one workgroup per row ------------------------------------------------------------
__device__ __forceinline__ int8_t quantize_one(float v, float scale) {
    const float r = rintf(v / scale);  // round half to even (the default rounding mode)
    if (r != r) return 0;              // NaN: `clamp` keeps it and `as i8` makes it 0
    return (int8_t)fminf(fmaxf(r, -127.0f), 127.0f);
}

__global__ __launch_bounds__(256) void quantize_rows_kernel(const float *__restrict__ x, int64_t k, int8_t *__restrict__ q,
                                                           float *__restrict__ scales) {
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const float *xr = x + row * k;
    float amax = 0.0f;
    for (int64_t i = threadIdx.x; i < k; i += 256) amax = fmaxf(amax, fabsf(xr[i]));  // f32::max skips NaN, as fmaxf does
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, kWave));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float scale = amax > 0.0f ? amax / 127.0f : 1.0f;
    if (threadIdx.x == 0) scales[row] = scale;
    int8_t *qr = q + row * k;
    for (int64_t i = threadIdx.x; i < k; i += 256) qr[i] = quantize_one(xr[i], scale);
}

// Rows of whole 128-bit vectors that fit the registers of a workgroup (k <= 1024 VPT): read once with 128-bit loads,
// written as packed bytes (one 32-bit store per four values).
template <int VPT>
__global__ __launch_bounds__(256) void quantize_rows_vec_kernel(const float *__restrict__ x, int64_t k, int8_t *__restrict__ q,
                                                               float *__restrict__ scales) {
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const float4 *xr = reinterpret_cast<const float4 *>(x + row * k);
    const int nvec = (int)(k / 4);
    float4 v[VPT];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = threadIdx.x + i * 256;
        if (c < nvec) {  // read once: non-temporal
            typedef float nat_f4 __attribute__((ext_vector_type(4)));
            const nat_f4 t = __builtin_nontemporal_load(reinterpret_cast<const nat_f4 *>(xr + c));
            v[i] = make_float4(t.x, t.y, t.z, t.w);
        } else {
            v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[i].x), fabsf(v[i].y)), fmaxf(fabsf(v[i].z), fabsf(v[i].w))));
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, kWave));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float scale = amax > 0.0f ? amax / 127.0f : 1.0f;
    if (threadIdx.x == 0) scales[row] = scale;
    uint32_t *qr = reinterpret_cast<uint32_t *>(q + row * k);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = threadIdx.x + i * 256;
        if (c < nvec) {
            const uint32_t b0 = (uint8_t)quantize_one(v[i].x, scale), b1 = (uint8_t)quantize_one(v[i].y, scale);
            const uint32_t b2 = (uint8_t)quantize_one(v[i].z, scale), b3 = (uint8_t)quantize_one(v[i].w, scale);
            __builtin_nontemporal_store(b0 | (b1 << 8) | (b2 << 16) | (b3 << 24), qr + c);
        }
    }
}

// ---- the product -------------------------------------------------------------------------------------
struct I8Args {
    const int8_t *a;  // [m, k] quantised activations
    const int8_t *b;  // [n, k] quantised weights
    const float *a_scales, *b_scales, *bias;
    float *c;  // [m, n]
    int64_t m, n, k;
    int tiles_m, tiles_n;
    int vec_store;  // n % 4 == 0 and a 16-byte aligned output: interior tiles may use 128-bit stores
};

// One wavefront-wide global -> LDS copy of 16 bytes per lane: scalar base, one unsigned 32-bit byte offset per lane (no
// 64-bit vector address arithmetic: vector instructions take issue cycles from the MFMAs). Inline assembly so that the
// compiler's wait-count insertion does not see an LDS write it cannot disambiguate; the kernel waits for its loads
// itself before each barrier.
__device__ __forceinline__ void load_to_lds_16(const int8_t *base, unsigned lane_off, unsigned lds_chunk) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(base),
                 "s"(__builtin_amdgcn_readfirstlane(lds_chunk))
                 : "memory", "m0");
}

// A pointer every lane holds the same value of, made a scalar for the compiler.
__device__ __forceinline__ const int8_t *uniform_ptr(const int8_t *ptr) {
    const uint64_t v = reinterpret_cast<uint64_t>(ptr);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<const int8_t *>(((uint64_t)hi << 32) | lo);
}

constexpr int kBK = 64;     // bytes of K per stage
constexpr int kGroup = 8;   // tiles are walked in kGroup x kGroup squares, one square at a time per XCD

// Calls f(integral_constant<int, 0>{}) ... f(integral_constant<int, N - 1>{}).
template <int N, int I = 0, typename F> __device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<N, I + 1>(f);
    }
}

template <int N> __device__ __forceinline__ void wait_vmcnt() {
    // s_waitcnt with only the vector-memory counter set: low four bits [3:0], high two bits [15:14]
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// TWM x TWN MFMA tiles (32 x 32 each) per wavefront, WM x WN wavefronts: a 32 TWM WM x 32 TWN WN output tile per workgroup.
// (2, 2, 2, 2): 128 x 128, two workgroups per compute unit, for problems with few tiles. (4, 4, 2, 2): 256 x 256 on four
// wavefronts, one per SIMD, 256 accumulator registers per lane: half the L2 -> LDS traffic and half the LDS reads per MFMA.
// (4, 2, 2, 4): the same 256 x 256 tile on eight wavefronts of 128 x 64, two per SIMD, so that one wavefront's barrier and
// load waits are covered by the other's MFMAs (three fragment reads per four MFMAs instead of two). The integer MFMA
// retires 65 536 operations in 32 cycles, so an LDS-fed loop is bound by fragment reads: measured on this chip with no
// global traffic at all, one 128-bit read per MFMA sustains half of the matrix peak, one per two MFMAs four fifths.
// NS: LDS stages in the ring; NS - 1 stages of loads are in flight under one stage of MFMAs (a ring of five, which takes all
// 160 KiB of the LDS, measured the same as four: 0.372 against 0.374 of the int8 peak at 8192 x 4096 x 4096).
template <int TWM, int TWN, int WM, int WN, int NS>
__global__ __launch_bounds__(WM *WN * 64, TWM * TWN * 16 <= 128 ? 2 : 1) void i8_gemm_kernel(const I8Args p) {
    constexpr int kStages = NS;
    // (second bound: wavefronts per SIMD the register allocation must allow -- two while the accumulators take at most 128 registers)
    constexpr int NW = WM * WN, NT = NW * 64;
    constexpr int BM = 32 * TWM * WM, BN = 32 * TWN * WN;
    constexpr int A_BYTES = BM * kBK, STAGE = (BM + BN) * kBK;
    constexpr int LDA = BM / 16 / NW, LDB = BN / 16 / NW;  // load instructions per operand per wavefront per stage (16 rows each)
    constexpr int LPS = LDA + LDB;                         // load instructions per stage per wavefront
    static_assert(BM % (16 * NW) == 0 && BN % (16 * NW) == 0, "a wavefront loads whole 16-row pieces of each operand");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];  // [kStages][A | B]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    // Workgroup ids go round-robin over the 8 XCDs. Each XCD takes a contiguous run of the tile sequence, and the
    // sequence walks kGroup x kGroup squares of tiles, so the workgroups resident on one XCD at a time share a few
    // row panels of A and of B through that XCD's L2.
    int tile = blockIdx.x;
    {
        const int grid = (int)gridDim.x, per = grid / 8;
        if (per > 0 && tile < per * 8) tile = (tile % 8) * per + tile / 8;
    }
    int tile_m, tile_n;
    {
        const int band = kGroup * p.tiles_n;  // tiles in a band of kGroup tile rows
        const int b = tile / band, r = tile % band;
        const int rows = (p.tiles_m - b * kGroup) < kGroup ? (p.tiles_m - b * kGroup) : kGroup;  // the last band may be short
        const int sq = r / (rows * kGroup), rs = r % (rows * kGroup);
        tile_m = b * kGroup + rs % rows;
        tile_n = sq * kGroup + rs / rows;
    }
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;

    // Loader: one wavefront instruction covers 16 rows x 64 bytes; a wavefront loads BM / 4 rows of A and BN / 4 of B
    // per stage. Lane L -> row L / 4 of the 16, slot L % 4, fetched from the swizzled source slot so that the LDS
    // image is already swizzled.
    const unsigned lds0 = __builtin_amdgcn_readfirstlane((unsigned)reinterpret_cast<uintptr_t>(smem));
    const unsigned wave_u = __builtin_amdgcn_readfirstlane((unsigned)wave);
    const int lrow = lane >> 2, lslot = lane & 3;
    // Scalar tile bases and per-lane byte offsets from them (a tile spans at most 256 rows of k bytes: the launcher
    // checks that this fits 32 bits). Rows past the end repeat the last row; their results are not stored.
    const int64_t a_row0 = m0 < p.m ? m0 : p.m - 1, b_row0 = n0 < p.n ? n0 : p.n - 1;
    const int8_t *a_base = uniform_ptr(p.a + a_row0 * p.k), *b_base = uniform_ptr(p.b + b_row0 * p.k);
    unsigned a_off[LDA], b_off[LDB];
#pragma unroll
    for (int i = 0; i < LDA; ++i) {
        const int r = wave * (16 * LDA) + i * 16 + lrow;  // row inside the tile
        const int q = lslot ^ ((r >> 2) & 3);             // the logical slot that lives at physical slot lslot
        int64_t ar = m0 + r;
        ar = ar < p.m ? ar : p.m - 1;
        a_off[i] = (unsigned)((ar - a_row0) * p.k) + (unsigned)q * 16u;
    }
#pragma unroll
    for (int i = 0; i < LDB; ++i) {
        const int r = wave * (16 * LDB) + i * 16 + lrow;
        const int q = lslot ^ ((r >> 2) & 3);
        int64_t br = n0 + r;
        br = br < p.n ? br : p.n - 1;
        b_off[i] = (unsigned)((br - b_row0) * p.k) + (unsigned)q * 16u;
    }
    const int num_kt = (int)(p.k / kBK);
    auto issue = [&](int kt) __attribute__((always_inline)) {
        const unsigned base = lds0 + (unsigned)(kt % kStages) * STAGE;
        const int8_t *ak = a_base + (int64_t)kt * kBK, *bk = b_base + (int64_t)kt * kBK;  // scalar arithmetic
#pragma unroll
        for (int i = 0; i < LDA; ++i) load_to_lds_16(ak, a_off[i], base + wave_u * (LDA * 1024u) + i * 1024u);
#pragma unroll
        for (int i = 0; i < LDB; ++i) load_to_lds_16(bk, b_off[i], base + A_BYTES + wave_u * (LDB * 1024u) + i * 1024u);
    };

    V16i acc[TWM][TWN];
#pragma unroll
    for (int i = 0; i < TWM; ++i)
#pragma unroll
        for (int j = 0; j < TWN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

#pragma unroll
    for (int st = 0; st < kStages - 1; ++st)
        if (st < num_kt) issue(st);
    // Fragment addresses: lane (row = lane % 32 of a 32-row MFMA tile, k group = lane / 32). The swizzle term of a row
    // depends on lane % 32 only (tile rows of a wavefront start at multiples of 32), so two per-lane byte offsets per
    // operand - one for each 32-byte K step - serve every read, with the stage, the MFMA tile row and the operand as
    // immediate offsets: the loop below is unrolled over the ring of stages so that the stage index is a constant.
    const int frow = lane & 31, kg = lane >> 5;
    const unsigned swz = (unsigned)(frow >> 2) & 3u;
    unsigned fa[2], fb[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        const unsigned slot = ((unsigned)(ks * 2 + kg) ^ swz) << 4;
        fa[ks] = (unsigned)(wm * (32 * TWM) + frow) * kBK + slot;
        fb[ks] = (unsigned)A_BYTES + (unsigned)(wn * (32 * TWN) + frow) * kBK + slot;
    }
    V4i af[2][TWM], bf[2][TWN];  // fragment registers of the two 32-byte K steps of a stage
    auto fetch = [&](auto stage_c, int ks) __attribute__((always_inline)) {
        constexpr int stage = decltype(stage_c)::value;
        const unsigned char *base = smem + stage * STAGE;
#pragma unroll
        for (int i = 0; i < TWM; ++i) af[ks][i] = *reinterpret_cast<const V4i *>(base + fa[ks] + i * 32 * kBK);
#pragma unroll
        for (int j = 0; j < TWN; ++j) bf[ks][j] = *reinterpret_cast<const V4i *>(base + fb[ks] + j * 32 * kBK);
    };
    auto mma = [&](int ks) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TWM; ++i)
#pragma unroll
            for (int j = 0; j < TWN; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[ks][i], bf[ks][j], acc[i][j], 0, 0, 0);
    };
    // Stage s has landed for everybody once each wavefront has waited for its own loads of s and passed a barrier.
    auto land = [&](int s_) __attribute__((always_inline)) {
        // loads of the stages after s_ stay in flight: LPS instructions each, at most kStages - 2 stages
        const int younger = num_kt - 1 - s_;
        if (younger >= kStages - 2) wait_vmcnt<(kStages - 2) * LPS>();
        else if (kStages > 4 && younger == 2) wait_vmcnt<2 * LPS>();
        else if (younger == 1) wait_vmcnt<LPS>();
        else wait_vmcnt<0>();
        __syncthreads();
    };
    land(0);
    if (kStages - 1 < num_kt) issue(kStages - 1);
    fetch(std::integral_constant<int, 0>{}, 0);
    // Steady state, one stage per step: the fragments of a K step are read from LDS while the MFMAs of the step
    // before it run, across the stage boundary as well, so neither the LDS latency nor the barrier wait is followed
    // by an MFMA that needs what was just requested. A step is straight-line code (with a conditional fetch the
    // compiler's wait-count pass joins two paths in front of the second batch of MFMAs and makes it wait for the
    // reads that were only just issued); the last stage is finished after the loop.
    auto step = [&](int kt, auto stage_c) __attribute__((always_inline)) {
        constexpr int stage = decltype(stage_c)::value;
        fetch(stage_c, 1);
        mma(0);
        land(kt + 1);  // also: every wavefront has finished reading stage kt, whose buffer takes stage kt + kStages
        if (kt + kStages < num_kt) issue(kt + kStages);
        fetch(std::integral_constant<int, (stage + 1) % kStages>{}, 0);
        mma(1);
    };
    static_assert(kStages == 4 || kStages == 5, "the wait counts above cover rings of four and five stages");
    int kt = 0;
    for (; kt + kStages < num_kt; kt += kStages)
        static_for<kStages>([&](auto S) __attribute__((always_inline)) { step(kt + decltype(S)::value, S); });
    // one to kStages stages are left (kt is a multiple of kStages): all but the last as steps, then the last one's second half
    const int left = num_kt - kt;
    static_for<kStages - 1>([&](auto S) __attribute__((always_inline)) {
        if (left > decltype(S)::value + 1) step(kt + decltype(S)::value, S);
    });
    static_for<kStages>([&](auto S) __attribute__((always_inline)) {
        if (left == decltype(S)::value + 1) fetch(S, 1);
    });
    mma(0);
    mma(1);

    // Dequantise and store: lane owns column n = lane % 32 of each MFMA tile, rows 8 (r / 4) + 4 (lane / 32) + r % 4.
    // The row scales of the tile go through LDS (free by now): one coalesced load instead of 16 scattered loads per
    // MFMA tile row.
    __syncthreads();
    float *row_scale = reinterpret_cast<float *>(smem);
    for (int t = tid; t < BM; t += NT) row_scale[t] = (m0 + t < p.m) ? p.a_scales[m0 + t] : 0.0f;
    __syncthreads();
    const bool interior = m0 + BM <= p.m && n0 + BN <= p.n;  // no bounds tests on the common path
    const int64_t ldc = p.n;
    if (interior && p.vec_store) {
        // Interior tiles leave through LDS so that the output goes out in whole rows: in the accumulator a lane holds ONE
        // column, and storing from there writes 128-byte pieces; staged, a wavefront instruction writes 1 KiB of
        // consecutive columns per row with 128-bit stores. One slab per MFMA tile row i: the 32 rows of each wavefront
        // row, 32 WM x BN floats.
        float *stage = reinterpret_cast<float *>(smem) + BM;  // behind the row scales
        constexpr int V4 = BN / 4;                            // 128-bit vectors per output row
        constexpr int PASSES = 32 * WM * V4 / NT;
        static_assert(32 * WM * V4 % NT == 0, "a slab is a whole number of passes");
#pragma unroll
        for (int i = 0; i < TWM; ++i) {
            const int lrow0 = wm * (32 * TWM) + i * 32 + 4 * kg;  // tile row of accumulator element 0
            if (i > 0) __syncthreads();                           // the previous slab has been read
#pragma unroll
            for (int j = 0; j < TWN; ++j) {
                const int lcol = wn * (32 * TWN) + j * 32 + frow;
                const float ws = p.b_scales[n0 + lcol];
                const float bv = p.bias ? p.bias[n0 + lcol] : 0.0f;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int dr = 8 * (r >> 2) + (r & 3);
                    float y = (float)acc[i][j][r] * row_scale[lrow0 + dr] * ws;
                    if (p.bias) y += bv;
                    stage[(wm * 32 + 4 * kg + dr) * BN + lcol] = y;
                }
            }
            __syncthreads();
#pragma unroll
            for (int ps = 0; ps < PASSES; ++ps) {
                const int f = ps * NT + tid, srow = f / V4, c4 = f % V4;
                const float4 v = *reinterpret_cast<const float4 *>(stage + srow * BN + 4 * c4);
                float *dst = p.c + (m0 + (srow >> 5) * (32 * TWM) + i * 32 + (srow & 31)) * ldc + n0 + 4 * c4;
                typedef float nat_f4 __attribute__((ext_vector_type(4)));
                nat_f4 nv = {v.x, v.y, v.z, v.w};
                __builtin_nontemporal_store(nv, reinterpret_cast<nat_f4 *>(dst));
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < TWM; ++i) {
        const int lrow0 = wm * (32 * TWM) + i * 32 + 4 * kg;  // tile row of accumulator element 0
        float as_[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) as_[r] = row_scale[lrow0 + 8 * (r >> 2) + (r & 3)];
#pragma unroll
        for (int j = 0; j < TWN; ++j) {
            const int64_t col = n0 + wn * (32 * TWN) + j * 32 + frow;
            if (!interior && col >= p.n) continue;
            const float ws = p.b_scales[col];
            const float bv = p.bias ? p.bias[col] : 0.0f;
            float *c0 = p.c + (m0 + lrow0) * ldc + col;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int dr = 8 * (r >> 2) + (r & 3);
                if (interior || m0 + lrow0 + dr < p.m) {
                    float y = (float)acc[i][j][r] * as_[r] * ws;
                    if (p.bias) y += bv;
                    __builtin_nontemporal_store(y, c0 + dr * ldc);
                }
            }
        }
    }
}

template <int TWM, int TWN, int WM, int WN, int NS = 4> int32_t launch_i8_gemm(I8Args &p, hipStream_t st) {
    constexpr int BM = 32 * TWM * WM, BN = 32 * TWN * WN;
    constexpr size_t smem = (size_t)NS * (BM + BN) * kBK;  // 64 KiB (two workgroups per compute unit), 128 or 160 KiB (one)
    p.tiles_m = (int)fth::ceil_div(p.m, BM);
    p.tiles_n = (int)fth::ceil_div(p.n, BN);
    static bool attr_set = false;
    if (!attr_set) {
        FTH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(i8_gemm_kernel<TWM, TWN, WM, WN, NS>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)smem));
        attr_set = true;
    }
    i8_gemm_kernel<TWM, TWN, WM, WN, NS><<<dim3((unsigned)(p.tiles_m * p.tiles_n)), dim3(WM * WN * 64), smem, st>>>(p);
    FTH_CHECK_LAUNCH("i8_gemm");
    return FTH_OK;
}

// Any shape and alignment: one thread per output element.
__global__ __launch_bounds__(256) void i8_gemm_plain_kernel(const I8Args p) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= p.m * p.n) return;
    const int64_t row = idx / p.n, col = idx % p.n;
    const int8_t *a = p.a + row * p.k, *b = p.b + col * p.k;
    int acc = 0;
    for (int64_t i = 0; i < p.k; ++i) acc += (int)a[i] * (int)b[i];
    float y = (float)acc * p.a_scales[row] * p.b_scales[col];
    if (p.bias) y += p.bias[col];
    p.c[idx] = y;
}

int32_t quantize_entry(const float *x, int64_t rows, int64_t cols, int8_t *q, float *scales, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(rows >= 0 && cols >= 0, "quantize_i8: negative extent");
    if (rows == 0) return FTH_OK;
    FTH_ARG(scales && (cols == 0 || (x && q)), "quantize_i8: NULL operand");
    FTH_ARG(rows <= 2147483647LL, "quantize_i8: too many rows for one launch");
    hipStream_t st = fth::resolve_stream(s);
    const bool vec = cols % 4 == 0 && cols > 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0 && (reinterpret_cast<uintptr_t>(q) & 3u) == 0;
    if (vec && cols <= 1024) quantize_rows_vec_kernel<1><<<dim3((unsigned)rows), dim3(256), 0, st>>>(x, cols, q, scales);
    else if (vec && cols <= 2048) quantize_rows_vec_kernel<2><<<dim3((unsigned)rows), dim3(256), 0, st>>>(x, cols, q, scales);
    else if (vec && cols <= 4096) quantize_rows_vec_kernel<4><<<dim3((unsigned)rows), dim3(256), 0, st>>>(x, cols, q, scales);
    else if (vec && cols <= 8192) quantize_rows_vec_kernel<8><<<dim3((unsigned)rows), dim3(256), 0, st>>>(x, cols, q, scales);
    else quantize_rows_kernel<<<dim3((unsigned)rows), dim3(256), 0, st>>>(x, cols, q, scales);
    FTH_CHECK_LAUNCH("quantize_rows_i8");
    return FTH_OK;
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace

extern "C" {

int32_t fth_dev_quantize_rows_i8(const float *x, int64_t rows, int64_t cols, int8_t *q, float *scales, fth_stream s) {
    return quantize_entry(x, rows, cols, q, scales, s);
}

size_t fth_dev_linear_int8_workspace_bytes(int64_t m, int64_t k) {
    if (m <= 0 || k < 0) return 0;
    return align256((size_t)m * (size_t)k) + align256((size_t)m * sizeof(float));
}

int32_t fth_dev_linear_int8_prequantized_f32(const int8_t *x_i8, const float *a_scales, int64_t m, int64_t k, const int8_t *w_i8,
                                             const float *w_scales, int64_t n, const float *bias, float *out, fth_stream s) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(m >= 0 && n >= 0 && k >= 0, "linear_int8: negative extent");
    if (m == 0 || n == 0) return FTH_OK;
    FTH_ARG(a_scales && w_scales && out && (k == 0 || (x_i8 && w_i8)), "linear_int8: NULL operand");
    hipStream_t st = fth::resolve_stream(s);
    I8Args p;
    p.a = x_i8; p.b = w_i8; p.a_scales = a_scales; p.b_scales = w_scales; p.bias = bias; p.c = out;
    p.m = m; p.n = n; p.k = k;
    p.tiles_m = p.tiles_n = 0;
    p.vec_store = (n % 4 == 0 && (reinterpret_cast<uintptr_t>(out) & 15u) == 0) ? 1 : 0;
    const bool aligned = ((reinterpret_cast<uintptr_t>(x_i8) | reinterpret_cast<uintptr_t>(w_i8)) & 15u) == 0;
    const int64_t tiles128 = fth::ceil_div(m, 128) * fth::ceil_div(n, 128), tiles256 = fth::ceil_div(m, 256) * fth::ceil_div(n, 256);
    if (k >= kBK && k % kBK == 0 && k <= (1 << 23) && aligned && tiles128 <= 2147483647LL) {  // (256 rows of k bytes within 32 bits)
        // 256 x 256 tiles once they give every compute unit a workgroup and the reduction is long enough to pay for their
        // longer fill and drain: they need half the L2 -> LDS traffic per MFMA, and that path (about 27 bytes per clock
        // and compute unit in this access pattern) is what bounds the 128 x 128 loop. The choice depends on the shape only.
        const int cus = fth::compute_units() > 0 ? fth::compute_units() : 256;
        static const int forced = [] {
            const char *e = std::getenv("FT_HIP_I8_TILE");  // tuning knob: 128, 256 (four wavefronts) or 512 (256 x 256 on eight); else automatic
            return e ? std::atoi(e) : 0;
        }();
        const bool big = forced == 256 || forced == 512 || (forced != 128 && tiles256 >= cus && k >= 2048);
        int32_t rc;
        if (!big) rc = launch_i8_gemm<2, 2, 2, 2>(p, st);
        else if (forced == 256) rc = launch_i8_gemm<4, 4, 2, 2>(p, st);  // four wavefronts of 128 x 128 (kept for comparison)
        else rc = launch_i8_gemm<4, 2, 2, 4>(p, st);                     // eight wavefronts of 128 x 64, two per SIMD
        if (rc) return rc;
    } else {
        int64_t total;
        FTH_ARG(!__builtin_mul_overflow(m, n, &total) && fth::ceil_div(total, 256) <= 2147483647LL, "linear_int8: output too large for one launch");
        i8_gemm_plain_kernel<<<dim3((unsigned)fth::ceil_div(total, 256)), dim3(256), 0, st>>>(p);
        FTH_CHECK_LAUNCH("i8_gemm_plain");
    }
    return FTH_OK;
}

int32_t fth_dev_linear_int8_dynamic_f32(const float *x, int64_t m, int64_t k, const int8_t *w_i8, const float *w_scales, int64_t n,
                                        const float *bias, float *out, void *workspace, size_t workspace_bytes, fth_stream s) {
    FTH_ARG(m >= 0 && n >= 0 && k >= 0, "linear_int8_dynamic: negative extent");
    if (m == 0 || n == 0) return FTH_OK;
    const size_t need = fth_dev_linear_int8_workspace_bytes(m, k);
    FTH_ARG(workspace && workspace_bytes >= need, "linear_int8_dynamic: workspace of %zu bytes, %zu needed", workspace_bytes, need);
    int8_t *xq = static_cast<int8_t *>(workspace);
    float *scales = reinterpret_cast<float *>(static_cast<unsigned char *>(workspace) + align256((size_t)m * (size_t)k));
    if (int32_t rc = quantize_entry(x, m, k, xq, scales, s)) return rc;
    return fth_dev_linear_int8_prequantized_f32(xq, scales, m, k, w_i8, w_scales, n, bias, out, s);
}

}  // extern "C"
