// Fused fp32 scaled-dot-product-attention backward for gfx950: a query-owned statistics pass, a key-owned pass and a
// query-owned dQ pass (sdpa_backward_f32, crates/ft-kernel-cpu/src/lib.rs:5539-5650; the unit-dOut form :5662-5770).
//
// The reference materialises P = softmax(scale Q K^T) and dU per (batch, head) and runs five
// products around two row passes. Here the work is three launches on [num_bh, seq, D] operands,
// with the reference's five products and no sixth:
//   1. statistics, one workgroup per 128 queries walking the key tiles they can see: raw scores S = Q K^T and
//      dP = dOut V^T to HBM, and per row the log-sum-exp and delta = sum_j P_ij dP_ij (the reference's `dot`), both
//      from one online pass over the tiles                          (products S and dP);
//   2. one workgroup per block of 128 keys walking the query tiles it can see:
//      P = 2^(S c - lse), dS = P (dP - delta) written over dP,
//      dV += P^T dOut, dK += dS^T Q in registers                    (products dV and dK);
//   3. dQ = scale dS K with dS read in the accumulator layout of pass 2   (product dQ).
// P and dU never make the round trip through HBM between separate softmax and softmax-gradient row passes: per call S
// and dP are written once and read once, dS written once (in place of dP) and read once. A recompute design that keeps
// nothing in HBM needs eight to nine product passes; on fp32 matrix cores a product pass costs more than the HBM
// traffic it saves.
//
// MFMA layout of pass 2 (v_mfma_f32_32x32x2_f32; a wavefront owns 32 keys, the block's four wavefronts share
// each 32-query tile of Q and dOut through double-buffered LDS):
//   S and dP arrive from HBM in the accumulator layout of a [query, key] product: a lane holds ONE key (lane % 32) and
//   16 of the tile's 32 queries, so S, dP, lse, delta, P and dS are lane-local, and P / dS are the B operands of the
//   two products as they stand (MFMA step r contracts over exactly the two queries that register r holds):
//   dV^T[d, key]  += dOut_tile^T . P        A = dOut read along d (lane = d index)
//   dK^T[d, key]  += Q_tile^T . dS          A = Q read along d
// No atomics: each (key, d) of dK / dV is summed by one wavefront in query order, so runs are bitwise repeatable.

#include <cstdlib>
#include <type_traits>

#include "common.hpp"
#include "sdpa_bwd.hpp"

namespace {

constexpr int kWave = 64;
using Acc16 = float __attribute__((ext_vector_type(16)));
typedef float nat_f4 __attribute__((ext_vector_type(4)));

struct KeysArgs {
    const float *q, *dout, *s, *lse, *delta;
    float *dpds;  // dP in, dS out, element for element
    float *dk, *dv;
    int64_t num_bh, dout_bh_stride;
    int seq_q, seq_k;
    float scale;
    int causal;
    int row_block;  // dS is defined (zero where masked) from the start of the row block that holds a key block's first key; 0: from row 0
    int snake;      // > 0: every workgroup is resident at once; pass length of fth::snake_order
};

// One wavefront-wide global -> LDS copy of 16 bytes per lane (scalar base, per-lane byte offset): lane L's bytes land
// at lds_chunk + 16 L. Inline assembly so that the compiler's wait-count insertion does not see an LDS write it cannot
// disambiguate; the kernel waits for vmcnt(0) itself before each barrier.
__device__ __forceinline__ void load_to_lds_16(const float *base, unsigned lane_off, unsigned lds_chunk) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(base),
                 "s"(__builtin_amdgcn_readfirstlane(lds_chunk))
                 : "memory", "m0");
}

__device__ __forceinline__ void load_to_lds_4(const float *base, unsigned lane_off, unsigned lds_chunk) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1" ::"v"(lane_off), "s"(base),
                 "s"(__builtin_amdgcn_readfirstlane(lds_chunk))
                 : "memory", "m0");
}

template <int N> struct VecN;
template <> struct VecN<2> { using type = float2; };
template <> struct VecN<4> { using type = float4; };
__device__ __forceinline__ float vecn_get(const float2 &v, int e) { return e == 0 ? v.x : v.y; }
__device__ __forceinline__ float vecn_get(const float4 &v, int e) { return e == 0 ? v.x : e == 1 ? v.y : e == 2 ? v.z : v.w; }
__device__ __forceinline__ float f4_get(const float4 &v, int e) { return e == 0 ? v.x : e == 1 ? v.y : e == 2 ? v.z : v.w; }

// Workspace layout of the three score-shaped intermediates. Per (batch, head) the [seq_q, seq_k] plane is cut into
// 32 x 32 tiles of 4 KiB, tile (qt, kt) at tile index qt * KT + kt; partial tiles at the edges are stored whole.
// Inside a tile the 16-byte vector number (2 g + h) * 32 + c holds, for S and dP, the four elements
//   [row 8 g + 4 h + i][column c], i = 0..3     (the accumulator registers 4 g .. 4 g + 3 of lane 32 h + c when the
//                                                lanes run along the keys: what passes 1 and 2 hold), and for dS
//   [row c][column 8 g + 4 h + i], i = 0..3     (the B operand registers of lane 32 h + c of the dQ pass, whose lanes
//                                                run along the queries).
// Every access of every pass is then one 16-byte vector per lane and 1 KiB in one piece per instruction, except the dS
// stores of pass 2 (single elements, sixteen 16-byte pieces per instruction).
// S has QT tile rows. dP and dS share a slab of QT + 1 tile rows: dP tile (qt, kt) sits in tile row qt + 1 and dS
// tile (qt, kt) in tile row qt, so pass 2 writes the dS of a tile over the dP of the tile it finished before (every
// load of that one has long returned) and never over anything it has yet to read.
struct TileMap {
    unsigned qt_n, kt_n;
    __host__ __device__ TileMap(int seq_q, int seq_k) : qt_n((unsigned)(seq_q + 31) >> 5), kt_n((unsigned)(seq_k + 31) >> 5) {}
    __host__ __device__ int64_t s_slab_floats() const { return (int64_t)qt_n * kt_n * 1024; }
    __host__ __device__ int64_t d_slab_floats() const { return (int64_t)(qt_n + 1) * kt_n * 1024; }
    __host__ __device__ unsigned s_slab_bytes() const { return qt_n * kt_n * 4096u; }
    __host__ __device__ unsigned d_slab_bytes() const { return (qt_n + 1) * kt_n * 4096u; }
    __host__ __device__ unsigned row_bytes() const { return kt_n * 4096u; }  // one tile row
    __host__ __device__ unsigned tile_bytes(unsigned qt, unsigned kt) const { return (qt * kt_n + kt) * 4096u; }
    // byte offset of a lane's vector g = 0 inside a tile; vector g is 1024 g further on
    __host__ __device__ static unsigned lane_vec(int half, int c) { return (unsigned)(half * 32 + c) * 16u; }
};

// Reductions over the 32 lanes of each half of a wavefront, result in every lane: four data-parallel-primitive steps
// inside rows of 16 lanes (quad swaps, then the mirrored halves of 8 and of 16) and one swizzle across the two rows.
template <typename F> __device__ __forceinline__ float half_reduce(float x, F op) {
    auto dpp = [](float v, auto ctrl) __attribute__((always_inline)) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), decltype(ctrl)::value, 0xF, 0xF, true));
    };
    x = op(x, dpp(x, std::integral_constant<int, 0xB1>{}));   // quad_perm [1, 0, 3, 2]
    x = op(x, dpp(x, std::integral_constant<int, 0x4E>{}));   // quad_perm [2, 3, 0, 1]
    x = op(x, dpp(x, std::integral_constant<int, 0x141>{}));  // row_half_mirror
    x = op(x, dpp(x, std::integral_constant<int, 0x140>{}));  // row_mirror
    return op(x, __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, x), 0x401F)));  // lane ^ 16
}
__device__ __forceinline__ float half_max(float x) {
    return half_reduce(x, [](float a, float b) { return fmaxf(a, b); });
}
__device__ __forceinline__ float half_sum(float x) {
    return half_reduce(x, [](float a, float b) { return a + b; });
}

// ---------------------------------------------------------------------------------------------
// Statistics pass. One workgroup per 128 queries (a wavefront owns 32; a lane keeps the Q and dOut rows of query
// lane % 32 in registers as A operands), walking BC-key tiles of K and V through double-buffered LDS:
//   S[q, key]  = Q . K_tile^T,   dP[q, key] = dOut . V_tile^T      (the same product shape twice)
// In the accumulators a lane then holds ONE key column (lane % 32) of 16 of its wavefront's queries - the layout the
// key-owned pass reads - so a store instruction writes two whole 128-byte row segments. (With the operand roles the
// other way round a lane owns a query and its statistics need no exchange at all, but every store instruction then
// scatters thirty-two 32-byte pieces over as many rows; that variant ran 15% slower, and twice as slow with streaming
// stores, which shows what the L2 has to merge.) The price is that each lane keeps its own running (reference, sum,
// sum of P dP) triple for each of its 16 rows over the keys IT has seen; the 32 lanes of a row are merged once, at
// the end of the pass. A lane's reference 2^m moves only when one of its scores exceeds it by more than kLazy (log2
// units). Both tiles are read one 16-byte vector per lane with 16 consecutive lanes on 16 consecutive rows, so logical
// vector v of tile row r is stored in slot v ^ (r & 15) (the permutation applied on the global side of the copy).
// ---------------------------------------------------------------------------------------------
struct StatsArgs {
    const float *q, *k, *v, *dout;
    float *s, *dp, *lse, *delta;
    int64_t num_bh, dout_bh_stride;
    int seq_q, seq_k;
    float scale;
    int causal;
    int snake;  // > 0: every workgroup is resident at once; pass length of fth::snake_order
};

template <int D, int BC>
__global__ __launch_bounds__(256, 2) void sdpa_bwd_stats_kernel(const StatsArgs p) {
    constexpr int KS = BC / 32;        // 32-key sub-tiles per tile
    constexpr int VPR = D / 4;         // 16-byte vectors per row
    constexpr int RPC = 64 / VPR;      // tile rows per 1 KiB load instruction
    constexpr int CPW = BC / RPC / 4;  // load instructions per wavefront per operand tile
    constexpr int TILE = BC * D;       // floats per operand tile
    constexpr int NST = 2 * KS * 4;    // 16-byte stores per wavefront and tile
    static_assert(NST == 8 || NST == 16, "the end-of-tile wait is written for 8 or 16 stores");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    float *Ks = reinterpret_cast<float *>(smem_raw);  // [2][BC][D], swizzled
    float *Vs = Ks + 2 * TILE;                        // [2][BC][D], swizzled

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lq = lane & 31, half = lane >> 5;
    const int seq_q = p.seq_q, seq_k = p.seq_k;
    const int q_blocks = (seq_q + 127) / 128;
    // Query blocks are issued heaviest (latest) first across all heads, and when the head count allows it every query
    // block of a head lands on the same XCD, whose L2 then serves the head's K and V to all of them.
    int64_t bh;
    int unit;
    {
        const int64_t pid = blockIdx.x;
        if (p.num_bh % 8 == 0) {
            const int64_t xcd = pid % 8, per = p.num_bh / 8;
            const int64_t w = fth::snake_order(pid / 8, p.snake, (int64_t)q_blocks * per);
            unit = (int)(w / per);
            bh = (w % per) * 8 + xcd;
        } else {
            unit = (int)(pid / p.num_bh);
            bh = pid % p.num_bh;
        }
    }
    const int qb = q_blocks - 1 - unit;
    const int q_blk0 = qb * 128, q_wave0 = q_blk0 + 32 * wave, qi = q_wave0 + lq;
    const bool q_live = qi < seq_q;
    const float *Kg = p.k + bh * (int64_t)seq_k * D, *Vg = p.v + bh * (int64_t)seq_k * D;
    const float c2 = p.scale * 1.44269502162933349609375f;  // scale * log2(e)

    // ---- Q and dOut rows of query lane % 32 into registers: lane holds row[8 t + 4 half + e] ----
    float4 qr[D / 8], dor[D / 8];
    {
        const int qc = q_live ? qi : seq_q - 1;
        const float *qrow = p.q + (bh * (int64_t)seq_q + qc) * D + 4 * half;
        const float *drow = p.dout + bh * p.dout_bh_stride + (int64_t)qc * D + 4 * half;
#pragma unroll
        for (int t = 0; t < D / 8; ++t) {
            qr[t] = *reinterpret_cast<const float4 *>(qrow + 8 * t);
            dor[t] = *reinterpret_cast<const float4 *>(drow + 8 * t);
        }
    }

    int blk_last_q = q_blk0 + 127, wave_last_q = q_wave0 + 31;
    if (blk_last_q > seq_q - 1) blk_last_q = seq_q - 1;
    if (wave_last_q > seq_q - 1) wave_last_q = seq_q - 1;
    int k_end = seq_k;
    if (p.causal && blk_last_q + 1 < k_end) k_end = blk_last_q + 1;
    const int num_kt = (k_end + BC - 1) / BC;

    // ---- tile loader: this wavefront owns CPW 1 KiB chunks of each tile; lane L of chunk c covers tile row
    //      c RPC + L / VPR, physical vector slot L % VPR ----
    const unsigned lds0 = __builtin_amdgcn_readfirstlane((unsigned)reinterpret_cast<uintptr_t>(smem_raw));
    const unsigned wave_u = __builtin_amdgcn_readfirstlane((unsigned)wave);
    int ld_row[CPW];
    unsigned ld_col[CPW];
#pragma unroll
    for (int ci = 0; ci < CPW; ++ci) {
        const int trow = (wave * CPW + ci) * RPC + lane / VPR;
        const int slot = lane % VPR;
        ld_row[ci] = trow;
        ld_col[ci] = 16u * (unsigned)((slot & ~15) | ((slot ^ trow) & 15));  // the logical vector that lives in this slot
    }
    auto issue_tile = [&](int kt, int buf) __attribute__((always_inline)) {
        const int row0 = kt * BC;
        const unsigned kdst = lds0 + (unsigned)(buf * TILE * 4) + wave_u * (CPW * 1024u);
        const unsigned vdst = lds0 + (unsigned)((2 * TILE + buf * TILE) * 4) + wave_u * (CPW * 1024u);
#pragma unroll
        for (int ci = 0; ci < CPW; ++ci) {
            int row = row0 + ld_row[ci];
            row = row < seq_k ? row : seq_k - 1;  // rows past the end repeat the last one: their scores are masked
            const unsigned off = (unsigned)row * (unsigned)(D * 4) + ld_col[ci];
            load_to_lds_16(Kg, off, kdst + ci * 1024u);
            load_to_lds_16(Vg, off, vdst + ci * 1024u);
        }
    };

    // ---- S and dP go out in whole 32 x 32 tiles of 4 KiB (workspace layout, see TileMap): a lane's four registers
    //      r = 4 g .. 4 g + 3 are one 16-byte vector of the tile, a store instruction writes 1 KiB in one piece. Range-
    //      checked buffer stores: the tile row of a wavefront whose queries lie wholly past seq_q is outside the slab. ----
    constexpr unsigned kOut = 0x40000000u;
    constexpr int kRsrcFlags = 0x00020000;  // raw buffer, 32-bit data format
    const TileMap tm(seq_q, seq_k);
    const __amdgpu_buffer_rsrc_t rs_s = __builtin_amdgcn_make_buffer_rsrc(p.s + bh * tm.s_slab_floats(), 0, (int)tm.s_slab_bytes(), kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs_dp = __builtin_amdgcn_make_buffer_rsrc(p.dp + bh * tm.d_slab_floats(), 0, (int)tm.d_slab_bytes(), kRsrcFlags);
    const unsigned lane_st = TileMap::lane_vec(half, lq);
    const unsigned qt_wave = (unsigned)(q_blk0 >> 5) + wave_u;  // from the scalar copy of the wavefront index: stays scalar
    typedef unsigned u4v __attribute__((ext_vector_type(4)));

    // fragment read t of tile row lq: vector 2 t + half sits in slot (2 t) ^ lx (bits 1..3 take eight per-lane values,
    // bit 4 is 2 t's own), lx = half ^ (lq & 15)
    const int lx = half ^ (lq & 15);
    int frag[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) frag[u] = lq * D + 4 * (((2 * u) ^ lx) & 15);

    // Per lane and row: reference m (log2 units; a large finite negative start, so that a lane that never sees a key of
    // a row keeps weight zero without an inf - inf), sum l of 2^(s c - m), sum a of 2^(s c - m) dP.
    constexpr float kLazy = 6.0f, kNone = -1.0e30f;
    float m_run[16], l_run[16], a_run[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        m_run[r] = kNone;
        l_run[r] = 0.f;
        a_run[r] = 0.f;
    }

    if (num_kt > 0) issue_tile(0, 0);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): own tile parts have landed
    __syncthreads();

    auto tile_step = [&](const int kt, auto buf_c) __attribute__((always_inline)) {
        constexpr int buf = decltype(buf_c)::value;
        const int key0 = kt * BC;
        if (kt + 1 < num_kt) issue_tile(kt + 1, buf ^ 1);
        // A wavefront whose every query precedes this tile's first key has nothing to add.
        const bool wave_active = !p.causal || key0 <= wave_last_q;
        if (wave_active) {
            Acc16 s[KS], dp[KS];
#pragma unroll
            for (int j = 0; j < KS; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    s[j][r] = 0.f;
                    dp[j][r] = 0.f;
                }
            // One step = one 16-byte fragment and the four MFMAs it feeds; steps alternate between the two products. The
            // fragment of step st + 2 is requested before the MFMAs of step st (the scheduler, left alone, sinks every
            // read to just before its use and each group of four MFMAs then waits out the LDS latency).
            const float *kb = Ks + buf * TILE, *vb = Vs + buf * TILE;
            constexpr int NSTEP = (D / 8) * KS * 2;
            auto frag_at = [&](int st) __attribute__((always_inline)) {
                const int t = st / (2 * KS), j = (st >> 1) % KS;
                const int off = frag[t & 7] + j * 32 * D + 4 * ((2 * t) & 16);
                return *reinterpret_cast<const float4 *>(((st & 1) ? vb : kb) + off);
            };
            float4 fr[3];
            fr[0] = frag_at(0);
            fr[1] = frag_at(1);
#pragma unroll
            for (int st = 0; st < NSTEP; ++st) {
                if (st + 2 < NSTEP) fr[(st + 2) % 3] = frag_at(st + 2);
                __builtin_amdgcn_sched_barrier(0);
                const float4 f = fr[st % 3];
                const int t = st / (2 * KS), j = (st >> 1) % KS;
                if (st & 1) {
                    dp[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(dor[t].x, f.x, dp[j], 0, 0, 0);
                    dp[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(dor[t].y, f.y, dp[j], 0, 0, 0);
                    dp[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(dor[t].z, f.z, dp[j], 0, 0, 0);
                    dp[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(dor[t].w, f.w, dp[j], 0, 0, 0);
                } else {
                    s[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(qr[t].x, f.x, s[j], 0, 0, 0);
                    s[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(qr[t].y, f.y, s[j], 0, 0, 0);
                    s[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(qr[t].z, f.z, s[j], 0, 0, 0);
                    s[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(qr[t].w, f.w, s[j], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            // ---- raw scores and dP of this wavefront's 32 queries x the tile's keys: element r of sub-tile j is query
            //      q_wave0 + 8 (r / 4) + 4 half + r % 4 against key key0 + 32 j + lane % 32 ----
            const bool tail = key0 + BC > seq_k;  // uniform
#pragma unroll
            for (int j = 0; j < KS; ++j) {
                // (a second sub-tile that starts past the last key has no tile of its own: its stores go nowhere)
                const unsigned v = (KS > 1 && key0 + 32 * j >= seq_k) ? kOut : lane_st;
                const unsigned ts = tm.tile_bytes(qt_wave, (unsigned)(key0 >> 5) + j);
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    // (element by element through float temporaries: a bit cast applied to a vector element directly reads element 0)
                    const float s0 = s[j][4 * g + 0], s1 = s[j][4 * g + 1], s2 = s[j][4 * g + 2], s3 = s[j][4 * g + 3];
                    const float d0 = dp[j][4 * g + 0], d1 = dp[j][4 * g + 1], d2 = dp[j][4 * g + 2], d3 = dp[j][4 * g + 3];
                    const u4v sx = {__builtin_bit_cast(unsigned, s0), __builtin_bit_cast(unsigned, s1), __builtin_bit_cast(unsigned, s2),
                                    __builtin_bit_cast(unsigned, s3)};
                    const u4v dx = {__builtin_bit_cast(unsigned, d0), __builtin_bit_cast(unsigned, d1), __builtin_bit_cast(unsigned, d2),
                                    __builtin_bit_cast(unsigned, d3)};
                    __builtin_amdgcn_raw_buffer_store_b128(sx, rs_s, v + (unsigned)g * 1024u, ts, 0);
                    __builtin_amdgcn_raw_buffer_store_b128(dx, rs_dp, v + (unsigned)g * 1024u, ts + tm.row_bytes(), 0);
                }
            }
            // ---- online statistics, per lane and row ----
            const bool need_mask = (p.causal && key0 + BC - 1 > q_wave0) || tail;
            if (need_mask) {  // wavefront-uniform; selects, no per-element branches
#pragma unroll
                for (int j = 0; j < KS; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int key = key0 + 32 * j + lq, qrow = q_wave0 + 8 * (r >> 2) + 4 * half + (r & 3);
                        const bool hidden = (p.causal && key > qrow) | (key >= seq_k);
                        s[j][r] = hidden ? -__builtin_inff() : s[j][r];
                    }
            }
            // exponents against the lane's references; the references move (rarely) when one exceeds kLazy
            float big = -__builtin_inff();
#pragma unroll
            for (int j = 0; j < KS; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) big = fmaxf(big, __builtin_fmaf(s[j][r], c2, -m_run[r]));
            if (__any(big > kLazy)) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float mx = s[0][r];
#pragma unroll
                    for (int j = 1; j < KS; ++j) mx = fmaxf(mx, s[j][r]);
                    const float m_new = fmaxf(m_run[r], mx * c2);
                    const float alpha = __builtin_amdgcn_exp2f(m_run[r] - m_new);
                    l_run[r] *= alpha;
                    a_run[r] *= alpha;
                    m_run[r] = m_new;
                }
            }
#pragma unroll
            for (int j = 0; j < KS; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[j][r], c2, -m_run[r]));
                    l_run[r] += e;
                    a_run[r] = __builtin_fmaf(e, dp[j][r], a_run[r]);
                }
            // the stores of this tile may stay in flight; the copies issued before them may not (in-order completion;
            // the counter holds 63 at most)
            if constexpr (NST == 8) __builtin_amdgcn_s_waitcnt(0x0F78);
            else __builtin_amdgcn_s_waitcnt(0x4F70);
        } else {
            __builtin_amdgcn_s_waitcnt(0x0F70);
        }
        __syncthreads();
    };
    for (int kt = 0; kt < num_kt; kt += 2) {
        tile_step(kt, std::integral_constant<int, 0>{});
        if (kt + 1 < num_kt) tile_step(kt + 1, std::integral_constant<int, 1>{});
    }
    // ---- merge the 32 lanes of every row (lanes 0..31 and 32..63 hold different rows): common reference, then the two
    //      sums rescaled to it ----
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const float m_all = half_max(m_run[r]);
        const float w = __builtin_amdgcn_exp2f(m_run[r] - m_all);
        const float l = half_sum(l_run[r] * w), a = half_sum(a_run[r] * w);
        const int qrow = q_wave0 + 8 * (r >> 2) + 4 * half + (r & 3);
        if (lq == 0 && qrow < seq_q) {
            p.lse[bh * (int64_t)seq_q + qrow] = m_all + __builtin_amdgcn_logf(l);  // v_log_f32 is log2
            p.delta[bh * (int64_t)seq_q + qrow] = a / l;
        }
    }
}

template <int D> int32_t launch_stats(const StatsArgs &a, hipStream_t st) {
    constexpr int BC = D <= 64 ? 64 : 32;  // two workgroups per compute unit either way
    constexpr size_t smem = (size_t)2 * 2 * BC * D * sizeof(float);
    static bool attr_set = false;
    if (!attr_set) {
        FTH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(sdpa_bwd_stats_kernel<D, BC>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)smem));
        attr_set = true;
    }
    const int64_t grid = a.num_bh * fth::ceil_div(a.seq_q, 128);
    FTH_ARG(grid <= 2147483647LL, "sdpa backward: grid too large");
    StatsArgs b = a;
    b.snake = a.num_bh % 8 == 0 ? fth::snake_pass_length(sdpa_bwd_stats_kernel<D, BC>, 256, smem, grid, a.causal != 0) : 0;
    sdpa_bwd_stats_kernel<D, BC><<<dim3((unsigned)grid), dim3(256), smem, st>>>(b);
    FTH_CHECK_LAUNCH("sdpa_bwd_stats");
    return FTH_OK;
}

template <int D>
__global__ __launch_bounds__(256, D == 64 ? 3 : 2) void sdpa_bwd_keys_kernel(const KeysArgs p) {
    constexpr int NDT = D / 32;        // 32-wide d-tiles of dK^T / dV^T
    constexpr int VPR = D / 4;         // 16-byte vectors per row
    constexpr int RPC = 64 / VPR;      // tile rows per 1 KiB load instruction
    constexpr int CPW = 32 / RPC / 4;  // load instructions per wavefront per operand tile
    constexpr int TILE = 32 * D;       // floats per operand tile
    using VV = typename VecN<NDT>::type;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    float *Qs = reinterpret_cast<float *>(smem_raw);  // [2][32][D], row order
    float *Os = Qs + 2 * TILE;                        // [2][32][D], row order
    float *Ls = Os + 2 * TILE;                        // [2][2][64]: log-sum-exp and delta of the tile's queries (32 used)

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lq = lane & 31, half = lane >> 5;
    // key blocks in ascending order: under a causal mask the heaviest come first (or, when every workgroup is resident
    // at once, in the back-and-forth order of fth::snake_order over each XCD's ids)
    const int64_t pid = p.snake > 0 ? (int64_t)(blockIdx.x % 8) + 8 * fth::snake_order(blockIdx.x / 8, p.snake, gridDim.x / 8) : (int64_t)blockIdx.x;
    const int kb = (int)(pid / p.num_bh);
    const int64_t bh = pid % p.num_bh;
    const int seq_q = p.seq_q, seq_k = p.seq_k;
    const unsigned wave_u = __builtin_amdgcn_readfirstlane((unsigned)wave);  // scalar copy: what derives from it stays scalar
    const int key0 = kb * 128, kw0 = key0 + 32 * (int)wave_u, kw = kw0 + lq;
    const bool key_live = kw < seq_k;
    const float *Qg = p.q + bh * (int64_t)seq_q * D;
    const float *Og = p.dout + bh * p.dout_bh_stride;
    const float *Lg = p.lse + bh * (int64_t)seq_q, *Dg = p.delta + bh * (int64_t)seq_q;
    const float c2 = p.scale * 1.44269502162933349609375f;  // scale * log2(e): the statistics are in log2 units

    int q_lo = 0;
    if (p.causal) q_lo = p.row_block > 0 ? (key0 / p.row_block) * p.row_block : 0;
    const int ntiles = (seq_q - q_lo + 31) / 32;

    // ---- tile loader (Q and dOut rows q_lo + 32 t .. + 31, rows past the end clamped: their weights are zero) ----
    const unsigned lds0 = __builtin_amdgcn_readfirstlane((unsigned)reinterpret_cast<uintptr_t>(smem_raw));
    int ld_row[CPW];
#pragma unroll
    for (int ci = 0; ci < CPW; ++ci) ld_row[ci] = (wave * CPW + ci) * RPC + lane / VPR;
    const unsigned ld_col = 16u * (unsigned)(lane % VPR);  // byte offset inside a row
    auto issue_tile = [&](int t, int buf) __attribute__((always_inline)) {
        const int row0 = q_lo + 32 * t;
        const unsigned qdst = lds0 + (unsigned)(buf * TILE * 4) + wave_u * (CPW * 1024u);
        const unsigned odst = lds0 + (unsigned)((2 * TILE + buf * TILE) * 4) + wave_u * (CPW * 1024u);
#pragma unroll
        for (int ci = 0; ci < CPW; ++ci) {
            int row = row0 + ld_row[ci];
            row = row < seq_q ? row : seq_q - 1;
            const unsigned off = (unsigned)row * (unsigned)(D * 4) + ld_col;
            load_to_lds_16(Qg, off, qdst + ci * 1024u);
            load_to_lds_16(Og, off, odst + ci * 1024u);
        }
        if (wave_u < 2) {  // wavefront 0 brings the log-sum-exps, wavefront 1 the deltas: one dword per lane
            int row = row0 + lane;
            row = row < seq_q ? row : seq_q - 1;
            load_to_lds_4(wave_u == 0 ? Lg : Dg, 4u * (unsigned)row, lds0 + (unsigned)(4 * TILE * 4) + (unsigned)(buf * 512) + wave_u * 256u);
        }
    };

    // Both products read their A operand along d: elements d = NDT lq .. NDT lq + NDT - 1 of tile row
    // 8 (r / 4) + 4 half + r % 4; consecutive lanes read consecutive vectors of one row.
    const int avec = (4 * half) * D + NDT * lq;

    Acc16 dvT[NDT], dkT[NDT];
#pragma unroll
    for (int e = 0; e < NDT; ++e)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            dvT[e][r] = 0.f;
            dkT[e][r] = 0.f;
        }

    // ---- S and dP in, dS out through buffer instructions on whole 4 KiB tiles (TileMap). Their range check is what
    //      drops the request for "the tile after the last" and for tiles this wavefront does not use: kOut, the "nowhere"
    //      value of the uniform tile part of an offset, is 2^30, every valid offset stays below it (the launcher checks
    //      the slab sizes), and any sum with a kOut in it is out of range and below 2^32. ----
    constexpr unsigned kOut = 0x40000000u;
    constexpr int kRsrcFlags = 0x00020000;  // raw buffer, 32-bit data format
    const TileMap tm(seq_q, seq_k);
    const __amdgpu_buffer_rsrc_t rs_s =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.s) + bh * tm.s_slab_floats(), 0, (int)tm.s_slab_bytes(), kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs_d = __builtin_amdgcn_make_buffer_rsrc(p.dpds + bh * tm.d_slab_floats(), 0, (int)tm.d_slab_bytes(), kRsrcFlags);
    const unsigned lane_ld = TileMap::lane_vec(half, lq);
    // dS element [row, column lq] of a tile: vector (lq / 4) * 32 + row, component lq % 4; row = 8 (r / 4) + 4 half + r % 4
    const unsigned lane_st = (unsigned)(lq >> 2) * 512u + (unsigned)(lq & 3) * 4u + (unsigned)half * 64u;
    const unsigned kt_wave = (unsigned)(kw0 >> 5), qt_lo = (unsigned)(q_lo >> 5);
    const bool wave_dead = kw0 >= seq_k;  // no key of this wavefront exists: it has no tile column
    auto wave_hidden = [&](int t) __attribute__((always_inline)) { return p.causal && q_lo + 32 * t + 31 < kw0; };
    // a tile of which this wavefront masks nothing: every row and key exists, every query sees every key
    auto wave_plain = [&](int t) __attribute__((always_inline)) {
        const int qt = q_lo + 32 * t;
        return qt + 32 <= seq_q && kw0 + 32 <= seq_k && (!p.causal || qt >= kw0 + 31);
    };
    typedef unsigned u4v __attribute__((ext_vector_type(4)));

    // The scores and dP of a tile sit in one register set, filled a whole tile ahead: as soon as the four elements of a
    // group of the tile in hand have been turned into P and dS, their registers are the destination of the next tile's
    // group. dS goes out as it is made, WITHOUT the softmax scale: the dQ product applies it when it stores and dK is
    // scaled once when it is stored. Vector memory operations complete in issue order, and a tile issues its operand
    // copies for the next tile FIRST, then exactly 8 loads and 16 stores (8 loads and no store where the wavefront sees
    // nothing of the tile): the wait that ends a tile is vmcnt(24) (vmcnt(8)), which covers the copies and leaves the
    // rest in flight.
    float sv[16], dv[16];
    unsigned ld_tile = kOut;  // uniform tile part of the next loads
    auto aim_loads = [&](int t) __attribute__((always_inline)) {
        const bool none = t >= ntiles || wave_hidden(t) || wave_dead;
        ld_tile = none ? kOut : tm.tile_bytes(qt_lo + (unsigned)t, kt_wave);
    };
    auto request = [&](int g) __attribute__((always_inline)) {
        const u4v x = __builtin_amdgcn_raw_buffer_load_b128(rs_s, lane_ld + (unsigned)g * 1024u, ld_tile, 2);
        const u4v y = __builtin_amdgcn_raw_buffer_load_b128(rs_d, lane_ld + (unsigned)g * 1024u + tm.row_bytes(), ld_tile, 2);
        // (whole vectors are cast: a bit cast applied to a vector element directly reads element 0)
        const nat_f4 xf = __builtin_bit_cast(nat_f4, x), yf = __builtin_bit_cast(nat_f4, y);
        sv[4 * g + 0] = xf.x; sv[4 * g + 1] = xf.y; sv[4 * g + 2] = xf.z; sv[4 * g + 3] = xf.w;
        dv[4 * g + 0] = yf.x; dv[4 * g + 1] = yf.y; dv[4 * g + 2] = yf.z; dv[4 * g + 3] = yf.w;
    };

    if (ntiles > 0) issue_tile(0, 0);
    aim_loads(0);
#pragma unroll
    for (int g = 0; g < 4; ++g) request(g);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): own tile parts have landed
    __syncthreads();

    // fp32 MFMAs and ordinary vector instructions do not overlap on this part (a wavefront's stream of
    // v_mfma_f32_32x32x2_f32 slows by the full issue time of every VALU instruction placed between them, with one
    // wavefront per SIMD or two), and a vector memory instruction costs about 20 cycles of it, so what counts is the
    // NUMBER of non-MFMA instructions per tile. The loop body therefore carries no mask logic: a tile that needs masking
    // (the diagonal, the last rows, the last keys) first sets the scores of its hidden pairs to -inf, whose weight
    // 2^(-inf) is an exact zero, and then runs the same body.
    auto tile_step = [&](const int t, auto buf_c) __attribute__((always_inline)) {
        constexpr int buf = decltype(buf_c)::value;
        const int qt = q_lo + 32 * t;
        if (t + 1 < ntiles) issue_tile(t + 1, buf ^ 1);
        const unsigned st_tile = wave_dead ? kOut : tm.tile_bytes(qt_lo + (unsigned)t, kt_wave);
        aim_loads(t + 1);
        auto store_ds = [&](int r, float x) __attribute__((always_inline)) {
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, x), rs_d, lane_st + (unsigned)(8 * (r >> 2) + (r & 3)) * 16u,
                                                  st_tile, 0);
        };
        if (!wave_hidden(t)) {
            // the tile's statistics: log-sum-exp and delta of the four queries of each element group
            const float *stats = Ls + buf * 128 + 4 * half;
            float4 lse_g[4], del_g[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                lse_g[g] = *reinterpret_cast<const float4 *>(stats + 8 * g);
                del_g[g] = *reinterpret_cast<const float4 *>(stats + 64 + 8 * g);
            }
            if (!wave_plain(t)) {  // wavefront-uniform, a few tiles per key block
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int qi = qt + 8 * (r >> 2) + 4 * half + (r & 3);
                    const bool hidden = (p.causal && kw > qi) | (qi >= seq_q) | !key_live;
                    sv[r] = hidden ? -__builtin_inff() : sv[r];
                }
            }
            // ---- P, dS (lane-local) and the two output products, software-pipelined by hand: step r reads the LDS
            //      operands of element r + 1 and does its P / dS arithmetic among the MFMAs of element r, whose operands
            //      step r - 1 left in registers; the last step of each group of four requests the next tile's group. The
            //      scheduling fences keep the compiler from sinking reads and requests to just before their first use. ----
            const float *ob = Os + buf * TILE + avec, *qb = Qs + buf * TILE + avec;
            VV ov_c = *reinterpret_cast<const VV *>(ob), qv_c = *reinterpret_cast<const VV *>(qb);
            float pw_c = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[0], c2, -lse_g[0].x));
            float ds_c = pw_c * (dv[0] - del_g[0].x);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int rn = r + 1 < 16 ? r + 1 : 15;
                VV ov_n = ov_c, qv_n = qv_c;
                if (r + 1 < 16) {
                    ov_n = *reinterpret_cast<const VV *>(ob + (8 * (rn >> 2) + (rn & 3)) * D);
                    qv_n = *reinterpret_cast<const VV *>(qb + (8 * (rn >> 2) + (rn & 3)) * D);
                }
                __builtin_amdgcn_sched_barrier(0);
                float pw_n = 0.f, ds_n = 0.f;
                if (r + 1 < 16) {
                    pw_n = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[rn], c2, -f4_get(lse_g[rn >> 2], rn & 3)));
                    ds_n = pw_n * (dv[rn] - f4_get(del_g[rn >> 2], rn & 3));
                }
                store_ds(r, ds_c);
#pragma unroll
                for (int e = 0; e < NDT; ++e) {
                    dvT[e] = __builtin_amdgcn_mfma_f32_32x32x2f32(vecn_get(ov_c, e), pw_c, dvT[e], 0, 0, 0);
                    dkT[e] = __builtin_amdgcn_mfma_f32_32x32x2f32(vecn_get(qv_c, e), ds_c, dkT[e], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                // elements 4 g .. 4 g + 3 were all consumed by the end of step 4 g + 2 (step r computes element r + 1)
                if ((r & 3) == 3) request(r >> 2);
                ov_c = ov_n; qv_c = qv_n; pw_c = pw_n; ds_c = ds_n;
            }
            __builtin_amdgcn_s_waitcnt(0x4F78);  // vmcnt(24)
        } else {
            // every (query, key) of this wavefront's part of the tile is masked, and the dQ pass does not read it
#pragma unroll
            for (int g = 0; g < 4; ++g) request(g);
            __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8)
        }
        __syncthreads();
    };
    for (int t = 0; t < ntiles; t += 2) {
        tile_step(t, std::integral_constant<int, 0>{});
        if (t + 1 < ntiles) tile_step(t + 1, std::integral_constant<int, 1>{});
    }
    // ---- store: lane owns key kw, d = NDT rho + e with rho = 8 (r / 4) + 4 half + r % 4 ----
    if (key_live) {
        float *dvrow = p.dv + (bh * (int64_t)seq_k + kw) * D, *dkrow = p.dk + (bh * (int64_t)seq_k + kw) * D;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int rho = 8 * (r >> 2) + 4 * half + (r & 3);
            if constexpr (NDT == 4) {
                *reinterpret_cast<float4 *>(dvrow + 4 * rho) = make_float4(dvT[0][r], dvT[1][r], dvT[2][r], dvT[3][r]);
                *reinterpret_cast<float4 *>(dkrow + 4 * rho) =
                    make_float4(p.scale * dkT[0][r], p.scale * dkT[1][r], p.scale * dkT[2][r], p.scale * dkT[3][r]);
            } else {
                *reinterpret_cast<float2 *>(dvrow + 2 * rho) = make_float2(dvT[0][r], dvT[1][r]);
                *reinterpret_cast<float2 *>(dkrow + 2 * rho) = make_float2(p.scale * dkT[0][r], p.scale * dkT[1][r]);
            }
        }
    }
}

template <int D> int32_t launch_keys(const KeysArgs &a, hipStream_t st) {
    constexpr size_t smem = (size_t)2 * 2 * 32 * D * sizeof(float) + 2 * 2 * 64 * sizeof(float);
    static bool attr_set = false;
    if (!attr_set) {
        FTH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(sdpa_bwd_keys_kernel<D>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_set = true;
    }
    const int64_t k_blocks = fth::ceil_div(a.seq_k, 128), grid = a.num_bh * k_blocks;
    FTH_ARG(grid <= 2147483647LL, "sdpa backward: grid too large");
    KeysArgs b = a;
    b.snake = grid % 8 == 0 ? fth::snake_pass_length(sdpa_bwd_keys_kernel<D>, 256, smem, grid, a.causal != 0) : 0;
    sdpa_bwd_keys_kernel<D><<<dim3((unsigned)grid), dim3(256), smem, st>>>(b);
    FTH_CHECK_LAUNCH("sdpa_bwd_keys");
    return FTH_OK;
}

// ---------------------------------------------------------------------------------------------
// Query-owned pass: dQ = scale . dS . K. One workgroup per 128 queries (a wavefront owns 32), walking the 32-key tiles
// its queries can see; K tiles through double-buffered LDS (row order, read along d), dS straight from HBM:
// dQ^T[d, q] += K_tile^T . dS^T, where MFMA step r contracts over the two keys 8 (r / 4) + 4 half + r % 4 and a lane's
// B operand is dS[q = lane % 32][that key] - four 16-byte loads per lane and tile (the workspace tiles hold dS in
// exactly that order, 1 KiB in one piece per instruction), requested one tile ahead. The key-owned pass stored
// explicit zeros for the masked pairs of every tile on the diagonal, so this loop has no mask logic: a wavefront simply
// stops at the last tile its queries reach. 64 MFMAs (D = 128) per tile against 4 loads and 16 LDS reads, and hardly a
// vector instruction in between.
// ---------------------------------------------------------------------------------------------
struct DqArgs {
    const float *ds, *k;
    float *dq;
    int64_t num_bh;
    int seq_q, seq_k;
    float scale;
    int causal;
    int snake;  // > 0: every workgroup is resident at once; pass length of fth::snake_order
};

template <int D>
__global__ __launch_bounds__(256, 2) void sdpa_bwd_dq_kernel(const DqArgs p) {
    constexpr int NDT = D / 32;
    constexpr int VPR = D / 4;         // 16-byte vectors per row
    constexpr int RPC = 64 / VPR;      // tile rows per 1 KiB load instruction
    constexpr int CPW = 32 / RPC / 4;  // load instructions per wavefront per tile
    constexpr int TILE = 32 * D;       // floats per K tile
    using VV = typename VecN<NDT>::type;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    float *Ks = reinterpret_cast<float *>(smem_raw);  // [2][32][D], row order

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lq = lane & 31, half = lane >> 5;
    const int64_t pid = p.snake > 0 ? (int64_t)(blockIdx.x % 8) + 8 * fth::snake_order(blockIdx.x / 8, p.snake, gridDim.x / 8) : (int64_t)blockIdx.x;
    const int q_blocks = (p.seq_q + 127) / 128;
    const int qb = q_blocks - 1 - (int)(pid / p.num_bh);  // heaviest (latest) query blocks first under a causal mask
    const int64_t bh = pid % p.num_bh;
    const int seq_q = p.seq_q, seq_k = p.seq_k;
    const unsigned wave_u = __builtin_amdgcn_readfirstlane((unsigned)wave);  // scalar copy: what derives from it stays scalar
    const int q_blk0 = qb * 128, q_wave0 = q_blk0 + 32 * (int)wave_u, qi = q_wave0 + lq;
    const bool q_live = qi < seq_q;
    const float *Kg = p.k + bh * (int64_t)seq_k * D;

    int blk_last_q = q_blk0 + 127, wave_last_q = q_wave0 + 31;
    if (blk_last_q > seq_q - 1) blk_last_q = seq_q - 1;
    if (wave_last_q > seq_q - 1) wave_last_q = seq_q - 1;
    int k_end = seq_k;
    if (p.causal && blk_last_q + 1 < k_end) k_end = blk_last_q + 1;
    const int ntiles = (k_end + 31) / 32;

    // ---- K tile loader (rows past the last key clamped: their dS is read as zero) ----
    const unsigned lds0 = __builtin_amdgcn_readfirstlane((unsigned)reinterpret_cast<uintptr_t>(smem_raw));
    auto issue_tile = [&](int t, int buf) __attribute__((always_inline)) {
        const unsigned dst = lds0 + (unsigned)(buf * TILE * 4) + wave_u * (CPW * 1024u);
#pragma unroll
        for (int ci = 0; ci < CPW; ++ci) {
            int row = 32 * t + (wave * CPW + ci) * RPC + lane / VPR;
            row = row < seq_k ? row : seq_k - 1;
            load_to_lds_16(Kg, (unsigned)row * (unsigned)(D * 4) + 16u * (unsigned)(lane % VPR), dst + ci * 1024u);
        }
    };

    // ---- dS through range-checked buffer loads on whole 4 KiB tiles (TileMap): a lane's vector g of tile (its
    //      wavefront's query tile, key tile t) is dS[its query][keys 8 g + 4 half .. + 3]; "nowhere" for a tile the
    //      wavefront does not use ----
    constexpr unsigned kOut = 0x40000000u;
    const TileMap tm(seq_q, seq_k);
    const __amdgpu_buffer_rsrc_t rs_ds =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.ds) + bh * tm.d_slab_floats(), 0, (int)tm.d_slab_bytes(), 0x00020000);
    const unsigned lane_ds = TileMap::lane_vec(half, lq);
    const unsigned qt_wave = (unsigned)(q_wave0 >> 5);
    typedef unsigned u4v __attribute__((ext_vector_type(4)));
    auto wave_active = [&](int t) __attribute__((always_inline)) { return !p.causal || 32 * t <= wave_last_q; };
    auto load_ds = [&](int t, float4(&dst)[4]) __attribute__((always_inline)) {
        const bool none = t >= ntiles || !wave_active(t) || q_wave0 >= seq_q;
        const unsigned ts = none ? kOut : tm.tile_bytes(qt_wave, (unsigned)t);
        const bool tail = 32 * t + 32 > seq_k;  // uniform: columns past the last key count as zero whatever the tile holds
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            u4v x = __builtin_amdgcn_raw_buffer_load_b128(rs_ds, lane_ds + (unsigned)g * 1024u, ts, 2);
            if (tail && 32 * t + 8 * g + 4 * half >= seq_k) x = (u4v){0u, 0u, 0u, 0u};
            dst[g] = __builtin_bit_cast(float4, x);
        }
    };

    Acc16 acc[NDT];
#pragma unroll
    for (int e = 0; e < NDT; ++e)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[e][r] = 0.f;

    float4 ds_a[4], ds_b[4];
    if (ntiles > 0) issue_tile(0, 0);
    load_ds(0, ds_a);
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();

    const int kvec = (4 * half) * D + NDT * lq;  // K is in row order: elements d = NDT lq .. of tile row 8 g + 4 half + j
    auto tile_step = [&](const int t, auto buf_c, float4(&ds_cur)[4], float4(&ds_nx)[4]) __attribute__((always_inline)) {
        constexpr int buf = decltype(buf_c)::value;
        if (t + 1 < ntiles) issue_tile(t + 1, buf ^ 1);
        load_ds(t + 1, ds_nx);
        if (wave_active(t)) {
            // the K fragment of step r + 2 is requested before the MFMAs of step r (the scheduler, left alone, sinks each
            // read to just before its use and every group of MFMAs then waits out the LDS latency)
            const float *kb = Ks + buf * TILE + kvec;
            auto frag_at = [&](int r) __attribute__((always_inline)) {
                return *reinterpret_cast<const VV *>(kb + (8 * (r >> 2) + (r & 3)) * D);
            };
            VV fr[3];
            fr[0] = frag_at(0);
            fr[1] = frag_at(1);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                if (r + 2 < 16) fr[(r + 2) % 3] = frag_at(r + 2);
                __builtin_amdgcn_sched_barrier(0);
                const VV kv = fr[r % 3];
                const float w = f4_get(ds_cur[r >> 2], r & 3);
#pragma unroll
                for (int e = 0; e < NDT; ++e) acc[e] = __builtin_amdgcn_mfma_f32_32x32x2f32(vecn_get(kv, e), w, acc[e], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // Everything requested at the top of this tile (the K copies and the next tile's dS, a whole tile of MFMAs ago)
        // has landed by now. The explicit vmcnt(0) also tells the compiler's wait-count pass so: it does not see the
        // K copies (inline assembly) and would otherwise place a too strict wait in front of the next tile's first MFMA.
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
    };
    for (int t = 0; t < ntiles; t += 2) {
        tile_step(t, std::integral_constant<int, 0>{}, ds_a, ds_b);
        if (t + 1 < ntiles) tile_step(t + 1, std::integral_constant<int, 1>{}, ds_b, ds_a);
    }

    // ---- store: lane owns query qi, d = NDT rho + e with rho = 8 (r / 4) + 4 half + r % 4 ----
    if (q_live) {
        float *row = p.dq + (bh * (int64_t)seq_q + qi) * D;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int rho = 8 * (r >> 2) + 4 * half + (r & 3);
            if constexpr (NDT == 4)
                *reinterpret_cast<float4 *>(row + 4 * rho) =
                    make_float4(p.scale * acc[0][r], p.scale * acc[1][r], p.scale * acc[2][r], p.scale * acc[3][r]);
            else
                *reinterpret_cast<float2 *>(row + 2 * rho) = make_float2(p.scale * acc[0][r], p.scale * acc[1][r]);
        }
    }
}

template <int D> int32_t launch_dq(const DqArgs &a, hipStream_t st) {
    constexpr size_t smem = (size_t)2 * 32 * D * sizeof(float);
    const int64_t grid = a.num_bh * fth::ceil_div(a.seq_q, 128);
    FTH_ARG(grid <= 2147483647LL, "sdpa backward: grid too large");
    DqArgs b = a;
    b.snake = grid % 8 == 0 ? fth::snake_pass_length(sdpa_bwd_dq_kernel<D>, 256, smem, grid, a.causal != 0) : 0;
    sdpa_bwd_dq_kernel<D><<<dim3((unsigned)grid), dim3(256), smem, st>>>(b);
    FTH_CHECK_LAUNCH("sdpa_bwd_dq");
    return FTH_OK;
}

}  // namespace

namespace fth {

bool sdpa_backward_fused_applies(int64_t num_bh, int64_t seq_q, int64_t seq_k, int64_t d_k, int64_t d_v, float scale) {
    static const bool off = [] {
        const char *e = std::getenv("FT_HIP_SDPA_BWD_FUSED");  // tuning / testing knob: 0 keeps the materialising backward
        return e && std::atoi(e) == 0;
    }();
    if (off || d_k != d_v || (d_k != 64 && d_k != 128) || seq_q < 32 || seq_k < 32 || !(scale > 0.f)) return false;
    // byte offsets inside one (batch, head) slab of tiles stay below 2^30, and so do those inside its operands
    const int64_t qt = (seq_q + 31) / 32, kt = (seq_k + 31) / 32;
    return (qt + 4) * kt * 4096 < ((int64_t)1 << 30) && seq_q * d_k < (1 << 28) && seq_k * d_k < (1 << 28);
}

void sdpa_backward_fused_workspace(int64_t num_bh, int64_t seq_q, int64_t seq_k, int64_t *s_floats, int64_t *d_floats) {
    const int64_t qt = (seq_q + 31) / 32, kt = (seq_k + 31) / 32;
    *s_floats = num_bh * qt * kt * 1024;
    *d_floats = num_bh * (qt + 1) * kt * 1024;
}

int32_t sdpa_backward_stats_f32(const float *q, const float *k, const float *v, const float *dout, int64_t dout_bh_stride, int64_t num_bh,
                                int64_t seq_q, int64_t seq_k, int64_t d, float scale, int causal, float *s_out, float *dp_out,
                                float *lse_out, float *delta_out, hipStream_t st) {
    StatsArgs a;
    a.q = q; a.k = k; a.v = v; a.dout = dout;
    a.s = s_out; a.dp = dp_out; a.lse = lse_out; a.delta = delta_out;
    a.num_bh = num_bh; a.dout_bh_stride = dout_bh_stride;
    a.seq_q = (int)seq_q; a.seq_k = (int)seq_k;
    a.scale = scale; a.causal = causal;
    if (d == 128) return launch_stats<128>(a, st);
    if (d == 64) return launch_stats<64>(a, st);
    return fth::set_error(FTH_ERR_INVALID_ARGUMENT, "sdpa_backward_stats: head size %lld", (long long)d);
}

int32_t sdpa_backward_keys_f32(const float *q, const float *dout, int64_t dout_bh_stride, const float *s, const float *lse,
                               const float *delta, int64_t num_bh, int64_t seq_q, int64_t seq_k, int64_t d, float scale, int causal,
                               int64_t row_block, float *dpds, float *dk, float *dv, hipStream_t st) {
    KeysArgs a;
    a.q = q; a.dout = dout; a.s = s; a.lse = lse; a.delta = delta;
    a.dpds = dpds; a.dk = dk; a.dv = dv;
    a.num_bh = num_bh; a.dout_bh_stride = dout_bh_stride;
    a.seq_q = (int)seq_q; a.seq_k = (int)seq_k;
    a.scale = scale; a.causal = causal; a.row_block = (int)row_block;
    if (d == 128) return launch_keys<128>(a, st);
    if (d == 64) return launch_keys<64>(a, st);
    return fth::set_error(FTH_ERR_INVALID_ARGUMENT, "sdpa_backward_keys: head size %lld", (long long)d);
}

int32_t sdpa_backward_dq_f32(const float *ds, const float *k, int64_t num_bh, int64_t seq_q, int64_t seq_k, int64_t d, float scale,
                             int causal, float *dq, hipStream_t st) {
    DqArgs a;
    a.ds = ds; a.k = k; a.dq = dq;
    a.num_bh = num_bh; a.seq_q = (int)seq_q; a.seq_k = (int)seq_k;
    a.scale = scale; a.causal = causal;
    if (d == 128) return launch_dq<128>(a, st);
    if (d == 64) return launch_dq<64>(a, st);
    return fth::set_error(FTH_ERR_INVALID_ARGUMENT, "sdpa_backward_dq: head size %lld", (long long)d);
}

}  // namespace fth
