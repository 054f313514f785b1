// Fused scaled-dot-product attention forward for gfx950 (fp32 on v_mfma_f32_32x32x2_f32).
//
// replaces sdpa_forward_f32 / sdpa_forward_f64 (crates/ft-kernel-cpu/src/lib.rs:5200-5284,
// 4572-4651): scores = Q.K^T, scale AFTER the product, row softmax over the first
// limit = min(qi + 1, seq_k) keys when causal (all seq_k otherwise), entries past the limit are
// exactly zero, out = P.V. The reference materialises a [64, seq_k] score tile per block and
// normalises P before the second product; this kernel never materialises scores: it walks the
// keys in tiles of 32 or 64 with an online softmax (running max m, running sum l, rescaled
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
// Work order: a causal workgroup runs a long query block and then the matching short one, so all
// workgroups carry the same work; units are issued heaviest first across all heads; and a
// (batch, head) always lands on the same XCD when the head count is a multiple of 8.

#include <cstdlib>
#include <type_traits>

#include "common.hpp"
#include "devmath.hpp"

namespace {

constexpr int kWave = 64;
constexpr int kXcds = 8;
#ifndef FTH_SDPA_DIRECT
#define FTH_SDPA_DIRECT 1
#endif

using Acc16 = float __attribute__((ext_vector_type(16)));

struct SdpaArgs {
    const void *q, *k, *v;
    void *out;
    fth_sdpa_desc d;
    double scale;
    int q_blocks;
    const void *mask;        // additive [seq_q, seq_k] rows (row pitch seq_k), or NULL
    int64_t mask_bh_stride;  // 0: one mask for every (batch, head); else elements between consecutive bh
    int64_t group;           // query heads per K/V head (grouped-query attention), >= 1
    int mask_vec;            // mask rows can be read as aligned float4 (seq_k % 4 == 0, 16-byte aligned base and bh stride)
    int snake;               // > 0: every workgroup is resident at once; pass length of fth::snake_order
};

// exp(x - m) for x <= m as 2^((x - m) * log2 e) on the hardware exp2 unit: subtract, multiply,
// v_exp_f32. The subtraction is exact or nearly so; rounding the product costs a relative error of
// about |x - m| * 2^-24 in the result, i.e. < 1e-6 for every weight that is not already
// negligible, far inside the 2e-5 parity tolerance. x = -inf gives exactly 0.
__device__ __forceinline__ float exp_diff(float x, float m) {
    return __builtin_amdgcn_exp2f((x - m) * 1.44269502162933349609375f);
}

// One wavefront-wide global -> LDS copy of 16 bytes per lane: lane L's bytes land at
// lds_chunk + 16 * L. Inline assembly so that the compiler's wait-count insertion does not see an
// LDS write it cannot disambiguate (it would wait for the load before every LDS read); the kernel
// waits for vmcnt(0) itself before each barrier.
__device__ __forceinline__ void load_to_lds_16(const float *src, unsigned lds_chunk) {
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(__builtin_amdgcn_readfirstlane(lds_chunk))
                 : "memory", "m0");
}

// The same with a scalar base and one unsigned 32-bit byte offset per lane: the offsets of a tile's chunks do not
// change from tile to tile, so the per-tile address work is scalar.
__device__ __forceinline__ void load_to_lds_16(const float *base, unsigned lane_off, unsigned lds_chunk) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(base),
                 "s"(__builtin_amdgcn_readfirstlane(lds_chunk))
                 : "memory", "m0");
}

// x of lanes 0..31 and x of lanes 32..63, each broadcast to both halves (one v_permlane32_swap, no LDS round trip).
__device__ __forceinline__ void both_halves(float x, float &lo, float &hi) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    lo = __uint_as_float(r[0]);
    hi = __uint_as_float(r[1]);
}

template <int N> struct VecN;
template <> struct VecN<1> { using type = float; };
template <> struct VecN<2> { using type = float2; };
template <> struct VecN<4> { using type = float4; };
__device__ __forceinline__ float vecn_get(const float &v, int) { return v; }
__device__ __forceinline__ float vecn_get(const float2 &v, int e) { return e == 0 ? v.x : v.y; }
__device__ __forceinline__ float vecn_get(const float4 &v, int e) { return e == 0 ? v.x : e == 1 ? v.y : e == 2 ? v.z : v.w; }
__device__ __forceinline__ float f4_get(const float4 &v, int e) { return e == 0 ? v.x : e == 1 ? v.y : e == 2 ? v.z : v.w; }

// D: head size (32, 64, 128). NW: wavefronts per block (4 or 2); a block owns 32 * NW consecutive
// queries per pass. PAIR: causal balancing -- the block runs two passes, query block
// (q_blocks - 1 - p) and then query block p, so every block does the same amount of work.
// BC: keys per tile (32, or 64 for the small head sizes, which halves the barriers and the
// cross-lane softmax steps per key).
// DIRECT: K/V tiles go global -> LDS with global_load_lds (no staging registers, no LDS stores; the
// loads stay in flight under the MFMAs). A wavefront instruction fills 1 KiB of LDS in lane order,
// so the tiles are unpadded. V rows are read whole (consecutive lanes, consecutive d) and need
// nothing more. K rows are read one 16-byte vector per lane with 16 consecutive lanes on 16
// consecutive rows, which would all hit the same banks (the LDS serves such a read 16 lanes at a
// time over 64 banks); logical vector q of tile row r is therefore stored in slot q ^ (r & 15), the
// permutation being applied on the global side by choosing which vector each lane fetches. Rows
// past seq_k are clamped to the last row (their scores are masked, their weights are zero).
// MASK: an additive mask row is read for every (query, key) score, mask[bh * mask_bh_stride + qi * seq_k + key]
// (sdpa_forward_masked_f64, crates/ft-kernel-cpu/src/lib.rs:4661-4741): score * scale + mask, then the same softmax.
// KSPLIT (causal balancing for launches that are resident all at once; needs PAIR, four wavefronts, 64-key tiles, the direct
// layout and no mask): the block owns 64 queries per pass and its wavefronts are (query half, key half) -- wavefront w takes
// queries 32 (w % 2) .. and the 32-key sub-tile w / 2 of every tile -- so with the (long, short) pairing every wavefront of
// every block does the same number of sub-tiles and no wavefront is left alone on its SIMD at the end (a lone wavefront's
// score -> softmax -> output chain keeps the matrix unit about 0.6 busy). The two key halves of a query wavefront are merged
// through LDS after the tile loop, in fixed order. K is single-buffered here (the next K tile is requested behind a barrier
// that follows the score MFMAs and lands under the softmax and the output MFMAs), V double-buffered: 48 KiB per block,
// three blocks per compute unit.
template <int D, int NW, bool PAIR, int BC, bool DIRECT, bool MASK, int MINW = 2, bool KSPLIT = false>
__global__ __launch_bounds__(64 * NW, MINW) void sdpa_mfma_kernel(const SdpaArgs p) {
    constexpr int kBC = BC;
    constexpr int KS = BC / 32;        // 32-key sub-tiles per tile
    constexpr int KSW = KSPLIT ? 1 : KS;  // sub-tiles a wavefront multiplies per tile
    constexpr int NTH = 64 * NW;
    constexpr int QWV = KSPLIT ? NW / 2 : NW;  // wavefronts along the queries
    constexpr int BQ = 32 * QWV;
    constexpr int KBUFS = KSPLIT ? 1 : 2;
    static_assert(!KSPLIT || (PAIR && NW == 4 && BC == 64 && DIRECT && !MASK), "key split: see the conditions above");
    constexpr int NDT = D / 32;        // 32-wide d-tiles of the output
    constexpr int KP = DIRECT ? D : D + 4;  // K tile row pitch (padded: odd number of 16-byte vectors)
    constexpr int VP = DIRECT ? D : D + 8;  // V tile row pitch (padded: rows j and j+4 land 32 banks apart)
    static_assert(!DIRECT || D >= 64, "the direct layout assumes rows of at least 256 bytes");
    constexpr int KT = kBC * KP;       // floats per K tile
    constexpr int VT = kBC * VP;
    constexpr int NV = kBC * (D / 4) / NTH;  // float4 per thread per tile
    static_assert(kBC * (D / 4) % NTH == 0, "tile must divide over the block");
    using VV = typename VecN<NDT>::type;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    float *Ks = reinterpret_cast<float *>(smem_raw);  // [KBUFS][kBC][KP]
    float *Vs = Ks + KBUFS * KT;                      // [2][kBC][VP]

    const fth_sdpa_desc &d = p.d;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lq = lane & 31, half = lane >> 5;
    const int qw = KSPLIT ? (wave & (QWV - 1)) : wave;  // which 32 queries of the block
    const int ksp = KSPLIT ? wave / QWV : 0;             // which 32-key half of each tile

    // ---- which (bh, unit): a unit is a query block, or a (heavy, light) pair of them ----
    const int units = PAIR ? (p.q_blocks + 1) / 2 : p.q_blocks;
    int64_t bh;
    int unit;
    {
        // Units are issued heaviest first across ALL heads (unit index is the slow digit), and when the head count
        // allows it a K/V head, with every query head that reads it, always lands on the same XCD (one L2).
        const int64_t pid = blockIdx.x;
        const int64_t g = p.group, kv_heads = d.num_bh / g;
        if (kv_heads % kXcds == 0) {
            const int64_t xcd = pid % kXcds, per = d.num_bh / kXcds;
            int64_t w = pid / kXcds;
            w = fth::snake_order(w, p.snake, (int64_t)units * per);
            unit = (int)(w / per);
            const int64_t idx = w % per;
            bh = ((idx / g) * kXcds + xcd) * g + idx % g;
        } else {
            unit = (int)(pid / d.num_bh);
            bh = pid % d.num_bh;
        }
    }
    const int64_t b = bh / d.heads, h = bh % d.heads, hk = h / p.group;  // query head h reads K/V head h / group
    const float *Q = static_cast<const float *>(p.q) + b * d.q_batch_stride + h * d.q_head_stride;
    const float *K = static_cast<const float *>(p.k) + b * d.k_batch_stride + hk * d.k_head_stride;
    const float *Vg = static_cast<const float *>(p.v) + b * d.v_batch_stride + hk * d.v_head_stride;
    float *O = static_cast<float *>(p.out) + b * d.o_batch_stride + h * d.o_head_stride;
    const float *Mk = MASK ? static_cast<const float *>(p.mask) + bh * p.mask_bh_stride : nullptr;
    const float scale = (float)p.scale;
    const float c2 = scale * 1.44269502162933349609375f;  // scale * log2(e)

    const int qb_first = p.q_blocks - 1 - unit;  // the long rows of a causal problem first
    const int npass = (PAIR && unit != qb_first) ? 2 : 1;

    for (int pass = 0; pass < npass; ++pass) {
        const int qb = pass == 0 ? qb_first : unit;
        // Row indices inside one head fit 32 bits (the launcher checks seq_q, seq_k < 2^31).
        const int q_blk0 = qb * BQ;
        const int q_wave0 = q_blk0 + qw * 32;
        const int qi = q_wave0 + lq;  // this lane's query
        const int seq_q_i = (int)d.seq_q;
        const bool q_live = qi < seq_q_i;

        // ---- Q rows into registers: lane holds Q[qi][8t + 4*half + e] ----
        float4 qr[D / 8];
#pragma unroll
        for (int t = 0; t < D / 8; ++t) {
            qr[t] = q_live ? *reinterpret_cast<const float4 *>(Q + (int64_t)qi * d.q_row_stride + 8 * t + 4 * half)
                           : make_float4(0.f, 0.f, 0.f, 0.f);
        }

        // ---- key range ----
        int blk_last_q = q_blk0 + BQ - 1;
        if (blk_last_q > seq_q_i - 1) blk_last_q = seq_q_i - 1;
        int k_end = (int)d.seq_k;  // exclusive
        if (d.causal && blk_last_q + 1 < k_end) k_end = blk_last_q + 1;
        const int num_kt = (k_end + kBC - 1) / kBC;
        int wave_last_q = q_wave0 + 31;
        if (wave_last_q > seq_q_i - 1) wave_last_q = seq_q_i - 1;

        // Tile loader: thread owns column vector ld_c of rows ld_row + i * RS; everything that
        // changes per tile or per i is wavefront-uniform, so the per-lane address is one base.
        constexpr int RS = NTH / (D / 4);  // rows covered by one sweep of the block
        const int ld_row = tid / (D / 4), ld_c = tid % (D / 4);
        const int seq_k_i = (int)d.seq_k;
        float4 kst[DIRECT ? 1 : NV], vst[DIRECT ? 1 : NV];
        const float *kbase = K + (int64_t)ld_row * d.k_row_stride + 4 * ld_c;
        const float *vbase = Vg + (int64_t)ld_row * d.v_row_stride + 4 * ld_c;
        // Direct loader: this wavefront owns CPW 1 KiB chunks of each tile; lane L of chunk c covers
        // tile row c * RPC + L / VPR, vector slot L % VPR.
        constexpr int VPR = D / 4, RPC = 64 / VPR, CPW = kBC / RPC / NW;
        static_assert(!DIRECT || kBC % (RPC * NW) == 0, "tile rows must divide into chunks per wavefront");
        const unsigned lds0 = __builtin_amdgcn_readfirstlane((unsigned)reinterpret_cast<uintptr_t>(smem_raw));
        const unsigned wave_u = __builtin_amdgcn_readfirstlane((unsigned)wave);
        // Per-lane byte offsets of this wavefront's chunks inside any full tile (row pitches up to 2^22 elements: launcher check).
        unsigned k_off[DIRECT ? CPW : 1], v_off[DIRECT ? CPW : 1];
        if constexpr (DIRECT) {
#pragma unroll
            for (int ci = 0; ci < CPW; ++ci) {
                const int trow = (wave * CPW + ci) * RPC + lane / VPR;  // row inside the tile
                const int slot = lane % VPR;
                const int kq = (slot & ~15) | ((slot ^ trow) & 15);
                k_off[ci] = (unsigned)trow * (unsigned)d.k_row_stride * 4u + 16u * (unsigned)kq;
                v_off[ci] = (unsigned)trow * (unsigned)d.v_row_stride * 4u + 16u * (unsigned)slot;
            }
        }
        // (WANT_K / WANT_V: the key-split variant requests the two tiles at different points of a step)
        auto issue_part = [&](int kt, int buf, auto want_k, auto want_v) __attribute__((always_inline)) {
            constexpr bool WANT_K = decltype(want_k)::value, WANT_V = decltype(want_v)::value;
            if constexpr (DIRECT) {
                const int row_t0 = kt * kBC;
                const float *kb = K + (int64_t)row_t0 * d.k_row_stride, *vb = Vg + (int64_t)row_t0 * d.v_row_stride;  // uniform
                const unsigned kdst = lds0 + (unsigned)((KBUFS == 2 ? buf : 0) * KT * 4) + wave_u * (CPW * 1024u);
                const unsigned vdst = lds0 + (unsigned)((KBUFS * KT + buf * VT) * 4) + wave_u * (CPW * 1024u);
                if (row_t0 + kBC <= seq_k_i) {
#pragma unroll
                    for (int ci = 0; ci < CPW; ++ci) {
                        if constexpr (WANT_K) load_to_lds_16(kb, k_off[ci], kdst + ci * 1024u);
                        if constexpr (WANT_V) load_to_lds_16(vb, v_off[ci], vdst + ci * 1024u);
                    }
                } else {  // the last, partial tile: rows past the end re-read the last row (their scores are masked)
#pragma unroll
                    for (int ci = 0; ci < CPW; ++ci) {
                        const int trow = (wave * CPW + ci) * RPC + lane / VPR;
                        const int slot = lane % VPR;
                        const int kq = (slot & ~15) | ((slot ^ trow) & 15);
                        const int crow = row_t0 + trow < seq_k_i ? trow : seq_k_i - 1 - row_t0;
                        if constexpr (WANT_K)
                            load_to_lds_16(kb, (unsigned)crow * (unsigned)d.k_row_stride * 4u + 16u * (unsigned)kq, kdst + ci * 1024u);
                        if constexpr (WANT_V)
                            load_to_lds_16(vb, (unsigned)crow * (unsigned)d.v_row_stride * 4u + 16u * (unsigned)slot, vdst + ci * 1024u);
                    }
                }
            }
        };
        auto issue_tile = [&](int kt, int buf) __attribute__((always_inline)) { issue_part(kt, buf, std::true_type{}, std::true_type{}); };
        auto load_tile = [&](int kt) {
            if constexpr (DIRECT) return;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int row0 = kt * kBC + i * RS;  // uniform
                if (row0 + ld_row < seq_k_i) {
                    kst[i] = *reinterpret_cast<const float4 *>(kbase + (int64_t)row0 * d.k_row_stride);
                    vst[i] = *reinterpret_cast<const float4 *>(vbase + (int64_t)row0 * d.v_row_stride);
                } else {
                    kst[i] = make_float4(0.f, 0.f, 0.f, 0.f);
                    vst[i] = make_float4(0.f, 0.f, 0.f, 0.f);
                }
            }
        };
        float *ks_st = Ks + ld_row * KP + 4 * ld_c;
        float *vs_st = Vs + ld_row * VP + 4 * ld_c;
        auto store_tile = [&](int buf) {
            if constexpr (DIRECT) return;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                *reinterpret_cast<float4 *>(ks_st + buf * KT + i * RS * KP) = kst[i];
                *reinterpret_cast<float4 *>(vs_st + buf * VT + i * RS * VP) = vst[i];
            }
        };

        Acc16 o[NDT];
#pragma unroll
        for (int e = 0; e < NDT; ++e)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[e][r] = 0.f;
        constexpr float kLazy = 6.0f;
        float m_run = -__builtin_inff();
        float l_run = 0.f;

        if (num_kt > 0) {
            issue_tile(0, 0);
            load_tile(0);
            store_tile(0);
        }
        if constexpr (DIRECT) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): own tile parts have landed
        __syncthreads();

        // Direct layout: fragment read t of K row lq is slot (2t) ^ lx; bits 1..3 of it take eight per-lane values, bit 4
        // is 2t's own (lx < 16), so eight addresses plus immediates cover every read of every tile.
        const int lx = half ^ (lq & 15);
        const float *kfrag[DIRECT ? 8 : 1];
        if constexpr (DIRECT) {
#pragma unroll
            for (int u = 0; u < 8; ++u) kfrag[u] = Ks + (lq + 32 * ksp) * KP + 4 * (((2 * u) ^ lx) & 15);
        }
        // One tile of the loop; the LDS buffer index is a compile-time constant (the loop below alternates two copies),
        // so every LDS address of a tile is a per-lane base plus an immediate.
        auto tile_step = [&](const int kt, auto buf_c) __attribute__((always_inline)) {
            constexpr int buf = decltype(buf_c)::value;
            const int key0 = kt * kBC + 32 * ksp;  // first key of this wavefront's part of the tile
            // The other buffer was released by the barrier that ended the previous tile.
            if (kt + 1 < num_kt) {
                if constexpr (KSPLIT) issue_part(kt + 1, buf ^ 1, std::false_type{}, std::true_type{});
                else issue_tile(kt + 1, buf ^ 1);
            }
            // A wavefront whose every query precedes this tile's first key has nothing to add.
            const bool wave_active = (!d.causal || key0 <= wave_last_q) && key0 < seq_k_i;
            // ---- the tile's mask values, requested before the score MFMAs that hide their latency:
            //      lane (query qi) element r of sub-tile j is key key0 + 32 j + 8 (r / 4) + 4 half + r % 4 ----
            Acc16 mk[MASK ? KS : 1];
            if constexpr (MASK) {
                if (wave_active) {
                    const float *mrow = Mk + (int64_t)(q_live ? qi : 0) * seq_k_i;
#pragma unroll
                    for (int j = 0; j < KS; ++j)
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            const int key = key0 + 32 * j + 8 * g + 4 * half;
                            float4 mv = make_float4(0.f, 0.f, 0.f, 0.f);
                            if (p.mask_vec) {  // seq_k % 4 == 0: a group of four keys never straddles the row end
                                if (key < seq_k_i) mv = *reinterpret_cast<const float4 *>(mrow + key);
                            } else {
                                if (key + 0 < seq_k_i) mv.x = mrow[key + 0];
                                if (key + 1 < seq_k_i) mv.y = mrow[key + 1];
                                if (key + 2 < seq_k_i) mv.z = mrow[key + 2];
                                if (key + 3 < seq_k_i) mv.w = mrow[key + 3];
                            }
                            mk[j][4 * g + 0] = mv.x;
                            mk[j][4 * g + 1] = mv.y;
                            mk[j][4 * g + 2] = mv.z;
                            mk[j][4 * g + 3] = mv.w;
                        }
                }
            }
            // ---- S^T = K_tile . Q^T, one 32-key sub-tile per accumulator ----
            Acc16 s[KSW];
            if (wave_active) {
#pragma unroll
                for (int j = 0; j < KSW; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) s[j][r] = 0.f;
                const float *kp = Ks + buf * KT + lq * KP + 4 * half;  // staged layout
#pragma unroll
                for (int t = 0; t < D / 8; ++t) {
#pragma unroll
                    for (int j = 0; j < KSW; ++j) {
                        // direct layout: vector 2t + half of row lq sits in slot (2t + half) ^ (lq & 15) = 2t ^ lx
                        const float4 kv = DIRECT ? *reinterpret_cast<const float4 *>(kfrag[t & 7] + (KBUFS == 2 ? buf : 0) * KT + j * 32 * KP + 4 * ((2 * t) & 16))
                                                 : *reinterpret_cast<const float4 *>(kp + j * 32 * KP + 8 * t);
                        s[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.x, qr[t].x, s[j], 0, 0, 0);
                        s[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.y, qr[t].y, s[j], 0, 0, 0);
                        s[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.z, qr[t].z, s[j], 0, 0, 0);
                        s[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.w, qr[t].w, s[j], 0, 0, 0);
                    }
                }
            }
            // The next tile's global loads are issued here, after the score MFMAs and before the
            // softmax: their latency is covered by the softmax and the P.V MFMAs, and their address
            // temporaries cannot be handed the registers the score accumulator is about to claim
            // (which makes the compiler wait for every load in flight before the first MFMA).
            if (kt + 1 < num_kt) load_tile(kt + 1);
            if constexpr (KSPLIT) {
                // every wavefront has read the one K buffer: the next K tile may land in it (under the softmax and the
                // output MFMAs; the step's closing wait covers it)
                __syncthreads();
                if (kt + 1 < num_kt) issue_part(kt + 1, 0, std::true_type{}, std::false_type{});
            }
            if (wave_active) {
                // ---- scale, mask, online softmax (lane-local query) ----
                constexpr int kMine = 32 * KSW;  // keys of the tile this wavefront scores
                const bool need_mask = (d.causal && key0 + kMine - 1 > q_wave0) || (key0 + kMine > seq_k_i);
                float mt = -__builtin_inff(), m_new, alpha, psum = 0.f;
                const float *vp = Vs + buf * VT + (4 * half + 32 * ksp) * VP + NDT * lq;
                if constexpr (!MASK) {
                    // Positive scale (the launcher sends unmasked calls with any other scale to the generic
                    // kernel): the row max is taken on the raw scores (scaling by a positive constant keeps
                    // the order), and scale * log2(e) is folded into one FMA per score, 2^(s * c2 - m) with
                    // the running max m kept in those log2 units.
                    if (need_mask) {  // wavefront-uniform; selects, no per-element branches
#pragma unroll
                        for (int j = 0; j < KSW; ++j)
#pragma unroll
                            for (int r = 0; r < 16; ++r) {
                                const int key = key0 + 32 * j + 8 * (r >> 2) + 4 * half + (r & 3);
                                const bool hidden = (d.causal && key > qi) | (key >= seq_k_i);
                                s[j][r] = hidden ? -__builtin_inff() : s[j][r];
                            }
                    }
#pragma unroll
                    for (int j = 0; j < KSW; ++j)
#pragma unroll
                        for (int r = 0; r < 16; ++r) mt = fmaxf(mt, s[j][r]);
                    // fp32 MFMAs and vector instructions share issue cycles, so the bookkeeping is kept off the common
                    // path: the reference m of a query moves only when a score of this tile exceeds it by more than
                    // kLazy (log2 units; weights stay below 2^kLazy and O / l does not depend on m). Only then do the two
                    // halves of the wavefront exchange their maxima and the accumulators get rescaled; the row sum stays
                    // a per-lane partial sum until the end.
                    if (__any(mt * c2 > m_run + kLazy)) {
                        float mlo, mhi;
                        both_halves(mt, mlo, mhi);
                        m_new = fmaxf(m_run, fmaxf(mlo, mhi) * c2);
                        alpha = __builtin_amdgcn_exp2f(m_run - m_new);
#pragma unroll
                        for (int e = 0; e < NDT; ++e)
#pragma unroll
                            for (int r = 0; r < 16; ++r) o[e][r] *= alpha;
                        l_run *= alpha;
                        m_run = m_new;
                    }
                    const float neg_m = -m_run;
                    // ---- O^T += V_tile^T . P^T with the exponentials in the same instruction stream ----
#pragma unroll
                    for (int j = 0; j < KSW; ++j)
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[j][r], c2, neg_m));
                            psum += e;
                            const VV vv = *reinterpret_cast<const VV *>(vp + (32 * j + 8 * (r >> 2) + (r & 3)) * VP);
#pragma unroll
                            for (int ee = 0; ee < NDT; ++ee)
                                o[ee] = __builtin_amdgcn_mfma_f32_32x32x2f32(vecn_get(vv, ee), e, o[ee], 0, 0, 0);
                        }
                    l_run += psum;
                } else {
#pragma unroll
                    for (int j = 0; j < KS; ++j)
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            float x = s[j][r] * scale;
                            if constexpr (MASK) x += mk[j][r];
                            s[j][r] = x;
                        }
                    if (need_mask) {  // wavefront-uniform; selects, no per-element branches
#pragma unroll
                        for (int j = 0; j < KS; ++j)
#pragma unroll
                            for (int r = 0; r < 16; ++r) {
                                const int key = key0 + 32 * j + 8 * (r >> 2) + 4 * half + (r & 3);
                                const bool hidden = (d.causal && key > qi) | (key >= seq_k_i);
                                s[j][r] = hidden ? -__builtin_inff() : s[j][r];
                            }
                    }
#pragma unroll
                    for (int j = 0; j < KS; ++j)
#pragma unroll
                        for (int r = 0; r < 16; ++r) mt = fmaxf(mt, s[j][r]);
                    float mlo, mhi;
                    both_halves(mt, mlo, mhi);
                    mt = fmaxf(mlo, mhi);
                    m_new = fmaxf(m_run, mt);
                    // A mask can hide every key seen so far (m_new still -inf): the weights are then 0 and the state
                    // stays empty, instead of the NaN that exp(-inf - -inf) would carry into later tiles. A row with
                    // no visible key at all ends as 0 / 0 = NaN, which is what the reference returns for it.
                    const float m_ref = (MASK && m_new == -__builtin_inff()) ? 0.f : m_new;
                    alpha = exp_diff(m_run, m_ref);
                    if (__any(alpha != 1.0f)) {
#pragma unroll
                        for (int e = 0; e < NDT; ++e)
#pragma unroll
                            for (int r = 0; r < 16; ++r) o[e][r] *= alpha;
                    }
                    // ---- O^T += V_tile^T . P^T, exponentials inside the MFMA stream as above ----
#pragma unroll
                    for (int j = 0; j < KS; ++j)
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const float e = exp_diff(s[j][r], m_ref);
                            psum += e;
                            const VV vv = *reinterpret_cast<const VV *>(vp + (32 * j + 8 * (r >> 2) + (r & 3)) * VP);
#pragma unroll
                            for (int ee = 0; ee < NDT; ++ee)
                                o[ee] = __builtin_amdgcn_mfma_f32_32x32x2f32(vecn_get(vv, ee), e, o[ee], 0, 0, 0);
                        }
                    l_run = l_run * alpha + psum;
                    m_run = m_new;
                }
            }
            if (kt + 1 < num_kt) store_tile(buf ^ 1);
            if constexpr (DIRECT) __builtin_amdgcn_s_waitcnt(0x0F70);
            __syncthreads();
        };
        for (int kt = 0; kt < num_kt; kt += 2) {
            tile_step(kt, std::integral_constant<int, 0>{});
            if (kt + 1 < num_kt) tile_step(kt + 1, std::integral_constant<int, 1>{});
        }
        if constexpr (KSPLIT) {
            // ---- merge the two key halves of each query wavefront (fixed order: half 0, then half 1) ----
            // The tile buffers are free (the loop ends on a barrier). State of key half 1: the accumulators, the reference
            // m (per query, the same in both lane halves) and the per-lane partial row sum, all relative to m.
            float *mg = reinterpret_cast<float *>(smem_raw) + qw * ((NDT * 16 + 2) * 64) + lane;
            if (ksp == 1) {
#pragma unroll
                for (int e = 0; e < NDT; ++e)
#pragma unroll
                    for (int r = 0; r < 16; ++r) mg[(e * 16 + r) * 64] = o[e][r];
                mg[(NDT * 16) * 64] = m_run;
                mg[(NDT * 16 + 1) * 64] = l_run;
            }
            __syncthreads();
            if (ksp == 0) {
                const float m1 = mg[(NDT * 16) * 64], l1 = mg[(NDT * 16 + 1) * 64];
                const float m = fmaxf(m_run, m1);
                // a half that saw no key of a query (m = -inf, sums 0) weighs nothing; both empty only when there is no key at all
                const float a0 = (m_run == -__builtin_inff()) ? 0.f : __builtin_amdgcn_exp2f(m_run - m);
                const float a1 = (m1 == -__builtin_inff()) ? 0.f : __builtin_amdgcn_exp2f(m1 - m);
#pragma unroll
                for (int e = 0; e < NDT; ++e)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o[e][r] = o[e][r] * a0 + mg[(e * 16 + r) * 64] * a1;
                l_run = l_run * a0 + l1 * a1;
            }
            __syncthreads();  // the merge area is tile memory again in the next pass
        }
        {  // the two halves of the wavefront hold partial row sums of the same queries
            float llo, lhi;
            both_halves(l_run, llo, lhi);
            l_run = llo + lhi;
        }

        // ---- normalise and store: lane owns query qi, d = NDT * rho + e ----
        if (q_live && ksp == 0) {
            float *orow = O + (int64_t)qi * d.o_row_stride;
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
    const int64_t b = bh / d.heads, h = bh % d.heads, hk = h / p.group;
    const T *Q = static_cast<const T *>(p.q) + b * d.q_batch_stride + h * d.q_head_stride + qi * d.q_row_stride;
    const T *K = static_cast<const T *>(p.k) + b * d.k_batch_stride + hk * d.k_head_stride;
    const T *V = static_cast<const T *>(p.v) + b * d.v_batch_stride + hk * d.v_head_stride;
    const T *mrow = p.mask ? static_cast<const T *>(p.mask) + bh * p.mask_bh_stride + qi * d.seq_k : nullptr;
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
            if (mrow) sc += mrow[key];
        }
        T mt = sc;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) mt = t_max(mt, __shfl_xor(mt, off, 64));
        const T m_new = t_max(m_run, mt);
        const T m_ref = (mrow && m_new == ninf) ? T(0) : m_new;  // every key so far hidden by the mask: empty state, not NaN
        const T alpha = t_exp(m_run - m_ref);
        const T pj = (key < limit) ? t_exp(sc - m_ref) : T(0);
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

// ---------------------------------------------------------------------------------------------
// fp64 on v_mfma_f64_16x16x4_f64 (sdpa_forward_f64, crates/ft-kernel-cpu/src/lib.rs:4572-4651, and the masked /
// grouped-query forms :4661-4850). The same scheme as the fp32 kernel at the shape of the fp64 MFMA: a wavefront
// owns 16 queries and a block of 4 wavefronts (64 queries) shares each tile of 16 keys through double-buffered LDS.
//   S^T[key, query] = K_tile . Q^T    16 x 16 accumulator: lane (query = lane % 16, g = lane / 16) holds keys
//                                     4 r + g, r = 0..3. The dot product over d_k is cut into four contiguous
//                                     ranges, one per lane group g (any split of the k index works as long as both
//                                     operands use it), so a lane's K and Q fragments are contiguous doubles:
//                                     128-bit LDS reads, and Q stays in registers for the whole kernel. Two
//                                     accumulators take alternate k steps, which halves the dependent MFMA chain.
//   O^T[d, query] += V_tile^T . P^T   MFMA step r contracts over keys 4 r + g, which is exactly what accumulator
//                                     element r of the lane holds: P is the B operand as it stands. Row i of
//                                     d-tile e is d = 32 (e / 2) + 2 i + e % 2, so one 128-bit read of V feeds two
//                                     d-tiles and a lane's outputs pair up into 16-byte stores.
// fp64 MFMAs and fp64 vector instructions share issue cycles (a vector instruction placed between two MFMAs delays the
// second by its full issue time, also with two wavefronts per SIMD), so the softmax is written for instruction count:
// Q is pre-multiplied by scale * log2(e) and the weights are 2^(x - ref) through an 18-instruction exp2; the reference
// ref of a query moves only when some score of the tile exceeds it by more than kLazy (then, and only then, the lane
// groups exchange their maxima and the accumulators are rescaled; weights stay below 2^kLazy, far from overflow, and the
// final O / l does not depend on ref); the row sum stays a per-lane partial sum until the end; the causal / tail
// selects run only in tiles that cross the diagonal or the end of the keys.
// ---------------------------------------------------------------------------------------------
using Acc4d = double __attribute__((ext_vector_type(4)));

template <int D, bool MASK>
__global__ __launch_bounds__(256, 2) void sdpa_mfma_f64_kernel(const SdpaArgs p) {
    constexpr int BC = 16;           // keys per tile
    constexpr int BQ = 64;           // queries per block
    constexpr int P = D + 2;         // LDS row pitch in doubles: 16 bytes of padding keep the 16 key rows of a fragment read on distinct banks
    constexpr int KT = BC * P;       // doubles per K (or V) tile
    constexpr int DQ = D / 4;        // doubles of a row that one lane group contracts over
    constexpr int NE = D / 16;       // d-tiles of the output
    constexpr int NV = BC * (D / 2) / 256;  // 16-byte vectors per thread per tile
    static_assert(BC * (D / 2) % 256 == 0 && NV >= 1, "tile must divide over the block");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    double *Ks = reinterpret_cast<double *>(smem_raw);  // [2][BC][P]
    double *Vs = Ks + 2 * KT;                           // [2][BC][P]

    const fth_sdpa_desc &d = p.d;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lq = lane & 15, g = lane >> 4;
    const int64_t pid = blockIdx.x;
    const int unit = (int)(pid / d.num_bh);  // heaviest (latest) query blocks first across all heads
    const int64_t bh = pid % d.num_bh;
    const int qb = p.q_blocks - 1 - unit;
    const int64_t b = bh / d.heads, h = bh % d.heads, hk = h / p.group;
    const double *Q = static_cast<const double *>(p.q) + b * d.q_batch_stride + h * d.q_head_stride;
    const double *K = static_cast<const double *>(p.k) + b * d.k_batch_stride + hk * d.k_head_stride;
    const double *Vg = static_cast<const double *>(p.v) + b * d.v_batch_stride + hk * d.v_head_stride;
    double *O = static_cast<double *>(p.out) + b * d.o_batch_stride + h * d.o_head_stride;
    const double *Mk = MASK ? static_cast<const double *>(p.mask) + bh * p.mask_bh_stride : nullptr;
    const double scale = p.scale;
    const int seq_q_i = (int)d.seq_q, seq_k_i = (int)d.seq_k;
    const int q_blk0 = qb * BQ, q_wave0 = q_blk0 + wave * 16, qi = q_wave0 + lq;
    const bool q_live = qi < seq_q_i;

    // Q: lane holds Q[qi][g * DQ + t], t = 0..DQ-1 (contiguous), times scale * log2(e): scores come out in log2 units
    const double qmul = scale * 1.4426950408889634074;
    double2 qr[DQ / 2];
#pragma unroll
    for (int t = 0; t < DQ / 2; ++t) {
        qr[t] = q_live ? *reinterpret_cast<const double2 *>(Q + (int64_t)qi * d.q_row_stride + g * DQ + 2 * t) : make_double2(0.0, 0.0);
        qr[t].x *= qmul;
        qr[t].y *= qmul;
    }

    int blk_last_q = q_blk0 + BQ - 1;
    if (blk_last_q > seq_q_i - 1) blk_last_q = seq_q_i - 1;
    int k_end = seq_k_i;
    if (d.causal && blk_last_q + 1 < k_end) k_end = blk_last_q + 1;
    const int num_kt = (k_end + BC - 1) / BC;
    int wave_last_q = q_wave0 + 15;
    if (wave_last_q > seq_q_i - 1) wave_last_q = seq_q_i - 1;

    // Tile loader through registers: thread owns vector column ld_c of rows ld_row + i * RS. Range-checked buffer loads:
    // the lane's byte offset is a constant, the tile and row-group part travels in the scalar offset, and rows past the
    // last key come back as zeros without a test (the range check covers the sum of both offsets).
    constexpr int RS = 256 / (D / 2);
    const int ld_row = tid / (D / 2), ld_c = tid % (D / 2);
    const __amdgpu_buffer_rsrc_t rs_k = __builtin_amdgcn_make_buffer_rsrc(const_cast<double *>(K), 0, (int)((unsigned)seq_k_i * (unsigned)d.k_row_stride * 8u), 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_v = __builtin_amdgcn_make_buffer_rsrc(const_cast<double *>(Vg), 0, (int)((unsigned)seq_k_i * (unsigned)d.v_row_stride * 8u), 0x00020000);
    const unsigned k_lane = ((unsigned)ld_row * (unsigned)d.k_row_stride + 2u * (unsigned)ld_c) * 8u;
    const unsigned v_lane = ((unsigned)ld_row * (unsigned)d.v_row_stride + 2u * (unsigned)ld_c) * 8u;
    const unsigned k_row_bytes = (unsigned)d.k_row_stride * 8u, v_row_bytes = (unsigned)d.v_row_stride * 8u;
    double2 kst[NV], vst[NV];
    auto load_tile = [&](int kt) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const unsigned row0 = (unsigned)(kt * BC + i * RS);  // uniform
            kst[i] = __builtin_bit_cast(double2, __builtin_amdgcn_raw_buffer_load_b128(rs_k, k_lane, row0 * k_row_bytes, 0));
            vst[i] = __builtin_bit_cast(double2, __builtin_amdgcn_raw_buffer_load_b128(rs_v, v_lane, row0 * v_row_bytes, 0));
        }
    };
    auto store_tile = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            *reinterpret_cast<double2 *>(Ks + buf * KT + (ld_row + i * RS) * P + 2 * ld_c) = kst[i];
            *reinterpret_cast<double2 *>(Vs + buf * KT + (ld_row + i * RS) * P + 2 * ld_c) = vst[i];
        }
    };

    Acc4d o[NE];
#pragma unroll
    for (int e = 0; e < NE; ++e) o[e] = (Acc4d){0.0, 0.0, 0.0, 0.0};
    const double ninf = -__builtin_inf();
    constexpr double kLazy = 6.0;  // log2 units
    double m_run = ninf, l_run = 0.0;

    if (num_kt > 0) {
        load_tile(0);
        store_tile(0);
    }
    __syncthreads();
    // One tile of the loop; the LDS buffer index is a compile-time constant (the loop below alternates two copies).
    auto tile_step = [&](const int kt, auto buf_c) __attribute__((always_inline)) {
        constexpr int buf = decltype(buf_c)::value;
        const int key0 = kt * BC;
        if (kt + 1 < num_kt) load_tile(kt + 1);  // in flight under this tile's matrix work
        const bool wave_active = !d.causal || key0 <= wave_last_q;
        if (wave_active) {
            // ---- the lane's four mask values, requested ahead of the score MFMAs ----
            double mk[4] = {0.0, 0.0, 0.0, 0.0};
            if constexpr (MASK) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int key = key0 + 4 * r + g;
                    if (q_live && key < seq_k_i) mk[r] = Mk[(int64_t)qi * seq_k_i + key];
                }
            }
            // ---- S^T = K_tile . Q^T ----
            Acc4d s0 = (Acc4d){0.0, 0.0, 0.0, 0.0}, s1 = s0;
            const double *kp = Ks + buf * KT + lq * P + g * DQ;
#pragma unroll
            for (int t = 0; t < DQ / 2; ++t) {
                const double2 kv = *reinterpret_cast<const double2 *>(kp + 2 * t);
                s0 = __builtin_amdgcn_mfma_f64_16x16x4f64(kv.x, qr[t].x, s0, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_f64_16x16x4f64(kv.y, qr[t].y, s1, 0, 0, 0);
            }
            // ---- mask, online softmax in log2 units (lane-local query; keys 4 r + g) ----
            double x[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                x[r] = s0[r] + s1[r];
                if constexpr (MASK) x[r] = __builtin_fma(mk[r], 1.4426950408889634074, x[r]);
            }
            if ((d.causal && key0 + BC - 1 > q_wave0) || key0 + BC > seq_k_i) {  // wavefront-uniform: the diagonal, the last keys
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int key = key0 + 4 * r + g;
                    const bool hidden = (d.causal && key > qi) | (key >= seq_k_i);
                    x[r] = hidden ? ninf : x[r];
                }
            }
            const double mt = fmax(fmax(x[0], x[1]), fmax(x[2], x[3]));
            if (__any(mt > m_run + kLazy)) {
                // some score outgrew the reference: the query's lane groups agree on a new one and rescale
                double mq = fmax(mt, __shfl_xor(mt, 16, kWave));
                mq = fmax(mq, __shfl_xor(mq, 32, kWave));
                const double m_new = fmax(m_run, mq);
                // Every key so far hidden (possible only under a mask): m_run stays -inf and the reference below is 0, so
                // the NaN of exp(-inf - -inf) never forms; a row with no visible key at all ends as 0 / 0 = NaN, as in
                // the reference.
                const double alpha = fth::exp2_softmax(m_run - ((m_new == ninf) ? 0.0 : m_new));
#pragma unroll
                for (int e = 0; e < NE; ++e)
#pragma unroll
                    for (int r = 0; r < 4; ++r) o[e][r] *= alpha;
                l_run *= alpha;
                m_run = m_new;
            }
            const double m_ref = (m_run == ninf) ? 0.0 : m_run;
            // ---- O^T += V_tile^T . P^T: step r contracts keys 4 r + g; d-tiles 2 e2 and 2 e2 + 1 share one read.
            //      Step r needs only weight r: the exponential of weight r + 1 sits between the MFMAs of step r. ----
            const double *vp = Vs + buf * KT + g * P + 2 * lq;
            double e_cur = fth::exp2_softmax(x[0] - m_ref);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const double e_r = e_cur;
                l_run += e_r;
                if (r + 1 < 4) e_cur = fth::exp2_softmax(x[r + 1] - m_ref);
#pragma unroll
                for (int e2 = 0; e2 < NE / 2; ++e2) {
                    const double2 vv = *reinterpret_cast<const double2 *>(vp + (4 * r) * P + 32 * e2);
                    o[2 * e2] = __builtin_amdgcn_mfma_f64_16x16x4f64(vv.x, e_r, o[2 * e2], 0, 0, 0);
                    o[2 * e2 + 1] = __builtin_amdgcn_mfma_f64_16x16x4f64(vv.y, e_r, o[2 * e2 + 1], 0, 0, 0);
                }
                if (r + 1 < 4) {
#pragma unroll
                    for (int i = 0; i < NE; ++i) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA of step r ...
                        __builtin_amdgcn_sched_group_barrier(0x002, (24 + NE - 1) / NE, 0);  // ... then a share of the next exponential
                    }
                }
            }
        }
        if (kt + 1 < num_kt) store_tile(buf ^ 1);
        __syncthreads();
    };
    for (int kt = 0; kt < num_kt; kt += 2) {
        tile_step(kt, std::integral_constant<int, 0>{});
        if (kt + 1 < num_kt) tile_step(kt + 1, std::integral_constant<int, 1>{});
    }

    // ---- normalise and store: element r of d-tile e is d = 32 (e / 2) + 2 (4 r + g) + e % 2 of query qi ----
    l_run += __shfl_xor(l_run, 16, kWave);  // the four lane groups of a query hold partial row sums
    l_run += __shfl_xor(l_run, 32, kWave);
    if (q_live) {
        double *orow = O + (int64_t)qi * d.o_row_stride;
#pragma unroll
        for (int e2 = 0; e2 < NE / 2; ++e2)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const double a0 = (num_kt > 0) ? o[2 * e2][r] / l_run : 0.0, a1 = (num_kt > 0) ? o[2 * e2 + 1][r] / l_run : 0.0;
                *reinterpret_cast<double2 *>(orow + 32 * e2 + 2 * (4 * r + g)) = make_double2(a0, a1);
            }
    }
}

template <int D> int32_t launch_mfma_f64(SdpaArgs &a, hipStream_t st) {
    constexpr size_t smem = (size_t)2 * 2 * 16 * (D + 2) * sizeof(double);
    a.q_blocks = (int)fth::ceil_div(a.d.seq_q, 64);
    const int64_t grid = a.d.num_bh * a.q_blocks;
    FTH_ARG(grid <= 2147483647LL, "sdpa: grid too large");
    if (a.mask) {
        static bool attr_set = false;
        if (!attr_set) {
            FTH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(sdpa_mfma_f64_kernel<D, true>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
            attr_set = true;
        }
        sdpa_mfma_f64_kernel<D, true><<<dim3((unsigned)grid), dim3(256), smem, st>>>(a);
    } else {
        static bool attr_set = false;
        if (!attr_set) {
            FTH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(sdpa_mfma_f64_kernel<D, false>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
            attr_set = true;
        }
        sdpa_mfma_f64_kernel<D, false><<<dim3((unsigned)grid), dim3(256), smem, st>>>(a);
    }
    FTH_CHECK_LAUNCH("sdpa_mfma_f64");
    return FTH_OK;
}

template <int D, int NW, bool PAIR, bool MASK, bool OCC3 = false, bool KSPLIT = false> int32_t launch_mfma_cfg(SdpaArgs &a, hipStream_t st) {
    // 64-key tiles where two workgroups still fit a CU; 32-key tiles (and a register budget for three) where three should;
    // the key-split variant: 64-key tiles, K single-buffered, three per CU
    constexpr int BC = KSPLIT ? 64 : OCC3 ? 32 : (D <= 64 && (NW == 4 || D <= 32)) ? 64 : 32;
    constexpr bool DIRECT = D >= 64 && FTH_SDPA_DIRECT;
    constexpr size_t smem = KSPLIT   ? (size_t)3 * BC * D * sizeof(float)
                            : DIRECT ? (size_t)2 * BC * 2 * D * sizeof(float)
                                     : (size_t)2 * BC * ((D + 4) + (D + 8)) * sizeof(float);
    auto kern = sdpa_mfma_kernel<D, NW, PAIR, BC, DIRECT, MASK, OCC3 ? 3 : 2, KSPLIT>;
    static bool attr_set = false;
    if (!attr_set) {
        FTH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    a.q_blocks = (int)fth::ceil_div(a.d.seq_q, KSPLIT ? 16 * NW : 32 * NW);
    const int64_t units = PAIR ? (a.q_blocks + 1) / 2 : a.q_blocks;
    const int64_t grid = a.d.num_bh * units;
    FTH_ARG(grid <= 2147483647LL, "sdpa: grid too large");
    a.snake = PAIR ? 0 : fth::snake_pass_length(kern, 64 * NW, smem, grid, a.d.causal != 0);
    kern<<<dim3((unsigned)grid), dim3(64 * NW), smem, st>>>(a);
    FTH_CHECK_LAUNCH("sdpa_mfma");
    return FTH_OK;
}

// ---------------------------------------------------------------------------------------------
// Small problems (the 128-token block: 4 heads x 128 queries): too few query blocks to fill the chip, so the time is a
// chain of latencies. A workgroup owns 32 queries and splits the KEYS over its four wavefronts (wavefront w takes the
// 32-key tiles w, w + 4, ...), each feeding the MFMAs straight from global memory (the operands are L2-resident; no LDS
// staging, no barrier in the loop), and the four partial (max, sum, output) states are merged through LDS in wavefront
// order. Same zero-shuffle S^T / P^T scheme and the same arithmetic per tile as sdpa_mfma_kernel.
template <int D>
__global__ __launch_bounds__(256) void sdpa_small_kernel(const SdpaArgs p) {
    constexpr int NDT = D / 32;
    constexpr int OP = D + 1;  // LDS row pitch of a partial output (odd: the 32 query rows land on distinct banks)
    using VV = typename VecN<NDT>::type;
    __shared__ float Os[4][32][OP];
    __shared__ float ms[4][32], ls[4][32];
    const fth_sdpa_desc &d = p.d;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lq = lane & 31, half = lane >> 5;
    const int64_t pid = blockIdx.x;
    const int qb = (int)(pid % p.q_blocks);
    const int64_t bh = pid / p.q_blocks;
    const int64_t b = bh / d.heads, h = bh % d.heads, hk = h / p.group;
    const float *Q = static_cast<const float *>(p.q) + b * d.q_batch_stride + h * d.q_head_stride;
    const float *K = static_cast<const float *>(p.k) + b * d.k_batch_stride + hk * d.k_head_stride;
    const float *Vg = static_cast<const float *>(p.v) + b * d.v_batch_stride + hk * d.v_head_stride;
    float *O = static_cast<float *>(p.out) + b * d.o_batch_stride + h * d.o_head_stride;
    const float c2 = (float)p.scale * 1.44269502162933349609375f;  // scale * log2(e); scale > 0 (launcher check)
    const int seq_q_i = (int)d.seq_q, seq_k_i = (int)d.seq_k;
    const int q0 = qb * 32, qi = q0 + lq;
    const bool q_live = qi < seq_q_i;

    float4 qr[D / 8];
#pragma unroll
    for (int t = 0; t < D / 8; ++t)
        qr[t] = q_live ? *reinterpret_cast<const float4 *>(Q + (int64_t)qi * d.q_row_stride + 8 * t + 4 * half) : make_float4(0.f, 0.f, 0.f, 0.f);

    int last_q = q0 + 31;
    if (last_q > seq_q_i - 1) last_q = seq_q_i - 1;
    int k_end = seq_k_i;
    if (d.causal && last_q + 1 < k_end) k_end = last_q + 1;
    const int num_kt = (k_end + 31) / 32;

    Acc16 o[NDT];
#pragma unroll
    for (int e = 0; e < NDT; ++e)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[e][r] = 0.f;
    float m_run = -__builtin_inff(), l_run = 0.f;

    for (int kt = wave; kt < num_kt; kt += 4) {
        const int key0 = kt * 32;
        int krow = key0 + lq;
        krow = krow < seq_k_i ? krow : seq_k_i - 1;  // rows past the end repeat the last one; their scores are masked
        const float *kp = K + (int64_t)krow * d.k_row_stride + 4 * half;
        Acc16 s;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
        for (int t = 0; t < D / 8; ++t) {
            const float4 kv = *reinterpret_cast<const float4 *>(kp + 8 * t);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.x, qr[t].x, s, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.y, qr[t].y, s, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.z, qr[t].z, s, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.w, qr[t].w, s, 0, 0, 0);
        }
        // V fragments of the tile, requested before the softmax that hides their latency
        VV vv[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            int vrow = key0 + 8 * (r >> 2) + (r & 3) + 4 * half;
            vrow = vrow < seq_k_i ? vrow : seq_k_i - 1;
            vv[r] = *reinterpret_cast<const VV *>(Vg + (int64_t)vrow * d.v_row_stride + NDT * lq);
        }
        float mt = -__builtin_inff();
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int key = key0 + 8 * (r >> 2) + 4 * half + (r & 3);
            const bool hidden = (d.causal && key > qi) | (key >= seq_k_i);
            s[r] = hidden ? -__builtin_inff() : s[r];
            mt = fmaxf(mt, s[r]);
        }
        float mlo, mhi;
        both_halves(mt, mlo, mhi);
        mt = fmaxf(mlo, mhi);
        const float m_new = fmaxf(m_run, mt * c2);
        // a wavefront's tiles can all lie past a query's causal limit (m_new still -inf): keep its state empty
        const float m_ref = (m_new == -__builtin_inff()) ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_ref);
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int e = 0; e < NDT; ++e)
#pragma unroll
                for (int r = 0; r < 16; ++r) o[e][r] *= alpha;
        }
        float psum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r], c2, -m_ref));
            psum += e;
#pragma unroll
            for (int ee = 0; ee < NDT; ++ee) o[ee] = __builtin_amdgcn_mfma_f32_32x32x2f32(vecn_get(vv[r], ee), e, o[ee], 0, 0, 0);
        }
        float plo, phi;
        both_halves(psum, plo, phi);
        l_run = l_run * alpha + (plo + phi);
        m_run = m_new;
    }

    // ---- merge the four partial states in wavefront order ----
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int rho = 8 * (r >> 2) + 4 * half + (r & 3);
#pragma unroll
        for (int e = 0; e < NDT; ++e) Os[wave][lq][NDT * rho + e] = o[e][r];
    }
    if (half == 0) {
        ms[wave][lq] = m_run;
        ls[wave][lq] = l_run;
    }
    __syncthreads();
    const int qf = tid & 31, dc = tid >> 5;  // query and one of eight d-chunks
    float m = ms[0][qf];
#pragma unroll
    for (int w = 1; w < 4; ++w) m = fmaxf(m, ms[w][qf]);
    float wgt[4], l = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        wgt[w] = (ms[w][qf] == -__builtin_inff()) ? 0.f : __builtin_amdgcn_exp2f(ms[w][qf] - m);
        l += ls[w][qf] * wgt[w];
    }
    if (q0 + qf < seq_q_i) {
        float *orow = O + (int64_t)(q0 + qf) * d.o_row_stride;
#pragma unroll
        for (int i = 0; i < D / 8; ++i) {
            const int dd = dc * (D / 8) + i;
            float acc = 0.f;
#pragma unroll
            for (int w = 0; w < 4; ++w) acc += Os[w][qf][dd] * wgt[w];
            orow[dd] = acc / l;
        }
    }
}

template <int D> int32_t launch_small_sdpa(SdpaArgs &a, hipStream_t st) {
    a.q_blocks = (int)fth::ceil_div(a.d.seq_q, 32);
    const int64_t grid = a.d.num_bh * a.q_blocks;
    sdpa_small_kernel<D><<<dim3((unsigned)grid), dim3(256), 0, st>>>(a);
    FTH_CHECK_LAUNCH("sdpa_small");
    return FTH_OK;
}

// Blocks of 128 queries (4 wavefronts) are used whenever they still give every other CU a
// workgroup; shorter problems fall back to blocks of 64 queries. Workgroups are issued heaviest
// first, which balances causal problems well enough that pairing a long with a short query
// block per workgroup (kept behind the tuning knob) measured no faster.
template <int D> int32_t launch_mfma(SdpaArgs &a, hipStream_t st) {
    bool pair = false;
    const int cus = fth::compute_units() > 0 ? fth::compute_units() : 256;
    const int64_t wg128 = a.d.num_bh * fth::ceil_div(a.d.seq_q, 128);
    bool wide = D >= 128 || 2 * wg128 >= (int64_t)cus;  // D = 128 staging does not fit 2-wavefront blocks
    static const int forced = [] {
        const char *e = std::getenv("FT_HIP_SDPA_CFG");  // tuning knob: bit 0 = 4 wavefronts, bit 1 = pairing, bit 2 = 32-key tiles at head size 64, bit 3 = key-split pairs at head size 64; -1 = auto
        return e ? std::atoi(e) : -1;
    }();
    if (forced >= 0) {
        wide = D >= 128 || (forced & 1);
        pair = a.d.causal != 0 && (forced & 2);
    }
    if constexpr (D == 64) {
        // Between two and four workgroups per compute unit a causal launch takes 32-key tiles, of which four workgroups
        // fit a compute unit (two of the 64-key ones do): everything is resident at once and the order of
        // fth::snake_order balances the compute units, which heaviest-first issue on two slots cannot (GPT-2's 96 heads
        // x 8 query blocks: the heaviest block alone is 8 of the 6.75 work units per slot).
        if constexpr (FTH_SDPA_DIRECT) {
            // More than two and at most three 128-query units per compute unit (GPT-2's 96 heads x S1024: exactly three): the
            // key-split pairs, every wavefront of every block the same length and all resident at once. Measured there: 126.8 ->
            // 119.2 us (0.647 -> 0.688 of the fp32 MFMA peak) against the unpaired blocks in the back-and-forth order.
            const bool split = forced >= 0 ? (forced & 8) != 0 : (wg128 > 2 * (int64_t)cus && wg128 <= 3 * (int64_t)cus);
            if (split && a.d.causal != 0 && !a.mask) return launch_mfma_cfg<D, 4, true, false, true, true>(a, st);
        }
        const bool three = forced >= 0 ? (forced & 4) != 0 : (a.d.causal != 0 && wg128 > 2 * (int64_t)cus && wg128 <= 4 * (int64_t)cus);
        if (!a.mask && !pair && wide && three) return launch_mfma_cfg<D, 4, false, false, true>(a, st);
    }
    if (a.mask) return wide ? launch_mfma_cfg<D, 4, false, true>(a, st) : launch_mfma_cfg<D, 2, false, true>(a, st);
    if (pair) return wide ? launch_mfma_cfg<D, 4, true, false>(a, st) : launch_mfma_cfg<D, 2, true, false>(a, st);
    return wide ? launch_mfma_cfg<D, 4, false, false>(a, st) : launch_mfma_cfg<D, 2, false, false>(a, st);
}

template <typename T>
int32_t sdpa_entry(const fth_sdpa_desc *d, double scale, const T *q, const T *k, const T *v, T *out, fth_stream s,
                   const T *mask = nullptr, int64_t mask_bh_stride = 0, bool masked = false) {
    FTH_REQUIRE_DEVICE();
    FTH_ARG(d != nullptr, "sdpa: desc is NULL");
    FTH_ARG(d->num_bh >= 0 && d->seq_q >= 0 && d->seq_k >= 0 && d->d_k >= 0 && d->d_v >= 0, "sdpa: negative extent");
    FTH_ARG(d->heads >= 1 && d->num_bh % d->heads == 0, "sdpa: heads (%lld) must divide num_bh (%lld)",
            (long long)d->heads, (long long)d->num_bh);
    const int64_t group = d->kv_group > 1 ? d->kv_group : 1;
    FTH_ARG(d->kv_group >= 0 && d->heads % group == 0, "sdpa: kv_group (%d) must divide heads (%lld)", (int)d->kv_group, (long long)d->heads);
    FTH_ARG(!masked || mask_bh_stride == 0 || mask_bh_stride >= d->seq_q * d->seq_k, "sdpa: mask_bh_stride %lld is neither 0 nor >= seq_q * seq_k",
            (long long)mask_bh_stride);
    if (d->num_bh == 0 || d->seq_q == 0 || d->d_v == 0) return FTH_OK;
    FTH_ARG(q && k && v && out, "sdpa: NULL operand");
    FTH_ARG(!masked || mask || d->seq_k == 0, "sdpa: NULL mask");
    FTH_ARG(d->seq_q < 2147483647LL - 256 && d->seq_k < 2147483647LL - 256, "sdpa: sequence too long");
    hipStream_t st = fth::resolve_stream(s);
    SdpaArgs a;
    a.q = q; a.k = k; a.v = v; a.out = out; a.d = *d; a.scale = scale;
    a.q_blocks = 0;  // set by the launcher of the chosen variant
    a.mask = masked ? mask : nullptr;
    a.mask_bh_stride = mask_bh_stride;
    a.group = group;
    a.snake = 0;
    a.mask_vec = (d->seq_k % 4 == 0 && mask_bh_stride % 4 == 0 && (reinterpret_cast<uintptr_t>(mask) & 15u) == 0) ? 1 : 0;
    auto al16 = [](const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; };
    auto m4 = [](int64_t x) { return x % 4 == 0; };
    if constexpr (std::is_same<T, float>::value) {
        const bool strides_ok = m4(d->q_batch_stride) && m4(d->q_head_stride) && m4(d->q_row_stride) &&
                                m4(d->k_batch_stride) && m4(d->k_head_stride) && m4(d->k_row_stride) &&
                                m4(d->v_batch_stride) && m4(d->v_head_stride) && m4(d->v_row_stride) &&
                                m4(d->o_batch_stride) && m4(d->o_head_stride) && m4(d->o_row_stride) &&
                                al16(q) && al16(k) && al16(v) && al16(out) &&
                                d->k_row_stride < (1 << 22) && d->v_row_stride < (1 << 22);  // a tile's lane offsets fit 32 bits
        // the unmasked MFMA kernels take the row maximum on the raw scores, which needs a positive scale
        if (strides_ok && d->d_k == d->d_v && d->seq_k > 0 && (masked || scale > T(0))) {
            // Too few 32-query blocks to give every compute unit one: the key-split kernel (one launch, no LDS staging)
            static const int small_knob = [] {
                const char *e = std::getenv("FT_HIP_SDPA_SMALL");  // tuning knob: 0 disables the small-problem kernel, 2 forces it
                return e ? std::atoi(e) : 1;
            }();
            const bool small_off = small_knob == 0;
            const int cus = fth::compute_units() > 0 ? fth::compute_units() : 256;
            if (!masked && !small_off && (small_knob == 2 || d->num_bh * fth::ceil_div(d->seq_q, 32) <= cus) && d->seq_k <= 4096) {
                if (d->d_k == 64) return launch_small_sdpa<64>(a, st);  // (128: the merge buffers would exceed 64 KiB of LDS)
                if (d->d_k == 32) return launch_small_sdpa<32>(a, st);
            }
            if (d->d_k == 128) return launch_mfma<128>(a, st);
            if (d->d_k == 64) return launch_mfma<64>(a, st);
            if (d->d_k == 32) return launch_mfma<32>(a, st);
        }
    }
    if constexpr (std::is_same<T, double>::value) {
        auto m2 = [](int64_t x) { return x % 2 == 0; };
        const bool strides_ok = m2(d->q_batch_stride) && m2(d->q_head_stride) && m2(d->q_row_stride) && m2(d->k_batch_stride) &&
                                m2(d->k_head_stride) && m2(d->k_row_stride) && m2(d->v_batch_stride) && m2(d->v_head_stride) &&
                                m2(d->v_row_stride) && m2(d->o_batch_stride) && m2(d->o_head_stride) && m2(d->o_row_stride) &&
                                al16(q) && al16(k) && al16(v) && al16(out);
        static const bool generic_only = [] {
            const char *e = std::getenv("FT_HIP_SDPA_F64_GENERIC");  // tuning / testing knob: 1 keeps fp64 on the generic kernel
            return e && std::atoi(e) != 0;
        }();
        // (the tile loads address a head's K and V through 32-bit byte offsets)
        const bool span_ok = (d->seq_k + 16) * d->k_row_stride < ((int64_t)1 << 28) && (d->seq_k + 16) * d->v_row_stride < ((int64_t)1 << 28);
        if (strides_ok && span_ok && d->d_k == d->d_v && d->seq_k > 0 && !generic_only) {
            if (d->d_k == 128) return launch_mfma_f64<128>(a, st);
            if (d->d_k == 64) return launch_mfma_f64<64>(a, st);
            if (d->d_k == 32) return launch_mfma_f64<32>(a, st);
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
    d->kv_group = 0;
}

int32_t fth_dev_sdpa_forward_f32(const fth_sdpa_desc *d, float scale, const float *q, const float *k, const float *v,
                                 float *out, fth_stream s) {
    return sdpa_entry<float>(d, (double)scale, q, k, v, out, s);
}

int32_t fth_dev_sdpa_forward_f64(const fth_sdpa_desc *d, double scale, const double *q, const double *k,
                                 const double *v, double *out, fth_stream s) {
    return sdpa_entry<double>(d, scale, q, k, v, out, s);
}

int32_t fth_dev_sdpa_forward_masked_f32(const fth_sdpa_desc *d, float scale, const float *q, const float *k, const float *v,
                                        const float *mask, int64_t mask_bh_stride, float *out, fth_stream s) {
    return sdpa_entry<float>(d, (double)scale, q, k, v, out, s, mask, mask_bh_stride, true);
}

int32_t fth_dev_sdpa_forward_masked_f64(const fth_sdpa_desc *d, double scale, const double *q, const double *k, const double *v,
                                        const double *mask, int64_t mask_bh_stride, double *out, fth_stream s) {
    return sdpa_entry<double>(d, scale, q, k, v, out, s, mask, mask_bh_stride, true);
}

}  // extern "C"
