// Fused key-owned and query-owned passes of the fp32 scaled-dot-product-attention backward for gfx950
// (sdpa_backward_f32, crates/ft-kernel-cpu/src/lib.rs:5539-5650; the unit-dOut form :5662-5770).
//
// The reference materialises P = softmax(scale Q K^T) and dU per (batch, head) and runs five
// products around two row passes. Here the work is three launches on [num_bh, seq, D] operands:
//   1. the forward kernel's preparation instantiation (csrc/sdpa.hip): raw scores S = Q K^T to
//      HBM, per-row log-sum-exp and delta = dOut . Out          (products S and P V);
//   2. this kernel, one workgroup per block of 128 keys walking the query tiles it can see:
//      P = 2^(S c - lse), dP = dOut V^T, dS = scale P (dP - delta) written to HBM,
//      dV += P^T dOut, dK += dS^T Q in registers                 (products dP, dV, dK);
//   3. a query-owned kernel, dQ = scale dS K with dS read in the accumulator layout of pass 2   (product dQ).
// Six product-sized MFMA passes instead of five, but P and dU never make the round trip through
// HBM between separate softmax and softmax-gradient row passes: per call S is written once and
// read once, dS written once and read once. A recompute design that keeps nothing in HBM needs
// eight to nine product passes (the statistics, then four in a key-owned and three in a
// query-owned kernel); on fp32 matrix cores a product pass costs more than the HBM traffic it saves.
//
// MFMA layout (v_mfma_f32_32x32x2_f32; a wavefront owns 32 keys, the block's four wavefronts share
// each 32-query tile of Q and dOut through double-buffered LDS):
//   dP[q, key]     = dOut_tile . V_blk^T    A = dOut rows from LDS (one 128-bit read feeds four MFMAs),
//                                           B = the wavefront's V rows, resident in registers.
//   In the accumulator a lane holds ONE key (lane % 32) and 16 of the tile's 32 queries, so S, lse,
//   delta, P and dS are lane-local, and P / dS are the B operands of the next two products as
//   they stand (MFMA step r contracts over exactly the two queries that register r holds):
//   dV^T[d, key]  += dOut_tile^T . P        A = dOut read along d (lane = d index)
//   dK^T[d, key]  += Q_tile^T . dS          A = Q read along d
// dOut is read in both directions, so its LDS image is XOR-swizzled (logical 16-byte vector v of
// tile row r in slot v ^ (r & 15)); Q is read along d only and stays in row order. No atomics:
// each (key, d) of dK / dV is summed by one wavefront in query order, so runs are bitwise repeatable.

#include <cstdlib>
#include <type_traits>

#include "common.hpp"
#include "sdpa_bwd.hpp"

namespace {

constexpr int kWave = 64;
using Acc16 = float __attribute__((ext_vector_type(16)));
typedef float nat_f4 __attribute__((ext_vector_type(4)));

struct KeysArgs {
    const float *q, *v, *dout, *s, *lse, *delta;
    float *ds, *dk, *dv;
    int64_t num_bh, dout_bh_stride;
    int seq_q, seq_k;
    float scale;
    int causal;
    int row_block;  // dS is defined (zero where masked) from the start of the row block that holds a key block's first key; 0: from row 0
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

template <int D>
__global__ __launch_bounds__(256, 1) void sdpa_bwd_keys_kernel(const KeysArgs p) {
    constexpr int NDT = D / 32;        // 32-wide d-tiles of dK^T / dV^T
    constexpr int VPR = D / 4;         // 16-byte vectors per row
    constexpr int RPC = 64 / VPR;      // tile rows per 1 KiB load instruction
    constexpr int CPW = 32 / RPC / 4;  // load instructions per wavefront per operand tile
    constexpr int TILE = 32 * D;       // floats per operand tile
    using VV = typename VecN<NDT>::type;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    float *Qs = reinterpret_cast<float *>(smem_raw);  // [2][32][D], row order
    float *Os = Qs + 2 * TILE;                        // [2][32][D], swizzled
    float *Ls = Os + 2 * TILE;                        // [2][2][64]: log-sum-exp and delta of the tile's queries (32 used)

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lq = lane & 31, half = lane >> 5;
    const int64_t pid = blockIdx.x;
    const int kb = (int)(pid / p.num_bh);  // key blocks in ascending order: under a causal mask the heaviest come first
    const int64_t bh = pid % p.num_bh;
    const int seq_q = p.seq_q, seq_k = p.seq_k;
    const int key0 = kb * 128, kw0 = key0 + 32 * wave, kw = kw0 + lq;
    const bool key_live = kw < seq_k;
    const int kc = key_live ? kw : seq_k - 1;
    const float *Qg = p.q + bh * (int64_t)seq_q * D;
    const float *Og = p.dout + bh * p.dout_bh_stride;
    const float *Sg = p.s + bh * (int64_t)seq_q * seq_k;
    float *DSg = p.ds + bh * (int64_t)seq_q * seq_k;
    const float *Lg = p.lse + bh * (int64_t)seq_q, *Dg = p.delta + bh * (int64_t)seq_q;
    const float c2 = p.scale * 1.44269502162933349609375f;  // scale * log2(e): the statistics are in log2 units

    // V rows of this lane's key: V[kc][8 t + 4 half + e]
    float4 vr[D / 8];
    {
        const float *vrow = p.v + (bh * (int64_t)seq_k + kc) * D + 4 * half;
#pragma unroll
        for (int t = 0; t < D / 8; ++t) vr[t] = *reinterpret_cast<const float4 *>(vrow + 8 * t);
    }

    int q_lo = 0;
    if (p.causal) q_lo = p.row_block > 0 ? (key0 / p.row_block) * p.row_block : 0;
    const int ntiles = (seq_q - q_lo + 31) / 32;

    // ---- tile loader (Q and dOut rows q_lo + 32 t .. + 31, rows past the end clamped: their weights are zero) ----
    const unsigned lds0 = __builtin_amdgcn_readfirstlane((unsigned)reinterpret_cast<uintptr_t>(smem_raw));
    const unsigned wave_u = __builtin_amdgcn_readfirstlane((unsigned)wave);
    int ld_row[CPW];
    unsigned q_col[CPW], o_col[CPW];  // byte offsets inside a row
#pragma unroll
    for (int ci = 0; ci < CPW; ++ci) {
        const int trow = (wave * CPW + ci) * RPC + lane / VPR;
        const int slot = lane % VPR;
        const int oq = (slot & ~15) | ((slot ^ trow) & 15);  // the logical vector that lives in physical slot `slot` of dOut's image
        ld_row[ci] = trow;
        q_col[ci] = 16u * (unsigned)slot;
        o_col[ci] = 16u * (unsigned)oq;
    }
    auto issue_tile = [&](int t, int buf) __attribute__((always_inline)) {
        const int row0 = q_lo + 32 * t;
        const unsigned qdst = lds0 + (unsigned)(buf * TILE * 4) + wave_u * (CPW * 1024u);
        const unsigned odst = lds0 + (unsigned)((2 * TILE + buf * TILE) * 4) + wave_u * (CPW * 1024u);
#pragma unroll
        for (int ci = 0; ci < CPW; ++ci) {
            int row = row0 + ld_row[ci];
            row = row < seq_q ? row : seq_q - 1;
            load_to_lds_16(Qg, (unsigned)row * (unsigned)(D * 4) + q_col[ci], qdst + ci * 1024u);
            load_to_lds_16(Og, (unsigned)row * (unsigned)(D * 4) + o_col[ci], odst + ci * 1024u);
        }
        if (wave_u < 2) {  // wavefront 0 brings the log-sum-exps, wavefront 1 the deltas: one dword per lane
            int row = row0 + lane;
            row = row < seq_q ? row : seq_q - 1;
            load_to_lds_4(wave_u == 0 ? Lg : Dg, 4u * (unsigned)row, lds0 + (unsigned)(4 * TILE * 4) + (unsigned)(buf * 512) + wave_u * 256u);
        }
    };

    // ---- per-lane LDS read offsets ----
    // dP product: 128-bit vector 2 t + half of tile row lq sits in slot (2 t) ^ lx (bits 1..3 take eight per-lane values,
    // bit 4 is 2 t's own), lx = half ^ (lq & 15).
    const int lx = half ^ (lq & 15);
    int ofrag[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) ofrag[u] = lq * D + 4 * (((2 * u) ^ lx) & 15);
    // dV product: elements d = NDT lq .. NDT lq + NDT - 1 of tile row qrow(r) = 8 (r / 4) + 4 half + r % 4
    int ovec[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int qrow = 8 * (r >> 2) + 4 * half + (r & 3);
        const int lv = (NDT * lq) / 4, within = (NDT * lq) % 4;
        ovec[r] = qrow * D + 4 * ((lv & ~15) | ((lv ^ qrow) & 15)) + within;
    }
    const int qvec = (4 * half) * D + NDT * lq;  // dK product: Q is in row order

    Acc16 dvT[NDT], dkT[NDT];
#pragma unroll
    for (int e = 0; e < NDT; ++e)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            dvT[e][r] = 0.f;
            dkT[e][r] = 0.f;
        }

    // ---- S in and dS out go through buffer instructions: their range check drops what lies past the end of the
    //      (batch, head) slab (rows past seq_q, the keys of dead lanes, the tile after the last, the store before the
    //      first), so no access needs a branch. A lane's byte offset is lane part + wavefront-uniform tile part + uniform
    //      row part; every valid sum stays below 2^30 (the launcher checks it) and kOut, the "nowhere" value of the lane
    //      and tile parts, is 2^30: any sum with a kOut in it is out of range and below 2^32. Lane and tile part travel in
    //      the instruction's vector offset (one add per tile), the row part in its scalar offset (none per row); the range
    //      check of this part covers the sum of both. ----
    constexpr unsigned kOut = 0x40000000u;
    constexpr int kRsrcFlags = 0x00020000;  // raw buffer, 32-bit data format
    const unsigned slab_bytes = (unsigned)seq_q * (unsigned)seq_k * 4u, row_bytes = (unsigned)seq_k * 4u;
    const __amdgpu_buffer_rsrc_t rs_s = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(Sg), 0, (int)slab_bytes, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs_ds = __builtin_amdgcn_make_buffer_rsrc(DSg, 0, (int)slab_bytes, kRsrcFlags);
    const unsigned lane_sd = key_live ? (unsigned)(4 * half) * row_bytes + 4u * (unsigned)kw : kOut;
    unsigned row_part[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) row_part[r] = (unsigned)(8 * (r >> 2) + (r & 3)) * row_bytes;
    auto wave_hidden = [&](int t) __attribute__((always_inline)) { return p.causal && q_lo + 32 * t + 31 < kw0; };
    // a tile of which this wavefront masks nothing: every row and key exists, every query sees every key
    auto wave_plain = [&](int t) __attribute__((always_inline)) {
        const int qt = q_lo + 32 * t;
        return qt + 32 <= seq_q && kw0 + 32 <= seq_k && (!p.causal || qt >= kw0 + 31);
    };

    // Two register sets of scores alternate: one is consumed by the tile in hand while the other receives the next
    // tile's (requested during this tile's dP product). dS is stored as it is made, WITHOUT the softmax scale: the dQ
    // product applies it as its alpha and dK is scaled once when it is stored. Vector memory operations complete in
    // issue order, and a tile issues its operand copies for the next tile FIRST, then exactly 16 score loads and 16 dS
    // stores: the wait that ends a tile is vmcnt(32), which covers the copies and leaves the rest in flight.
    float s_a[16], s_b[16];
    unsigned ld_tile = kOut;  // uniform tile part of the next loads
    auto aim_loads = [&](int t) __attribute__((always_inline)) {
        const unsigned qt = (unsigned)(q_lo + 32 * t);
        const bool none = t >= ntiles || wave_hidden(t);
        ld_tile = none ? kOut : qt * row_bytes;
    };

    if (ntiles > 0) issue_tile(0, 0);
    aim_loads(0);
#pragma unroll
    for (int r = 0; r < 16; ++r)
        s_a[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs_s, lane_sd + ld_tile + row_part[r], 0, 2));
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): own tile parts have landed
    __syncthreads();

    // fp32 MFMAs and ordinary vector instructions do not overlap on this part (a wavefront's stream of
    // v_mfma_f32_32x32x2_f32 slows by the full issue time of every VALU instruction placed between them, with one
    // wavefront per SIMD or two), so what counts is the NUMBER of non-MFMA instructions per tile. The loop body therefore
    // carries no mask logic: a tile that needs masking (the diagonal, the last rows, the last keys) first sets the scores
    // of its hidden pairs to -inf, whose weight 2^(-inf) is an exact zero, and then runs the same body.
    auto tile_step = [&](const int t, auto buf_c, float(&s_cur)[16], float(&s_nx)[16]) __attribute__((always_inline)) {
        constexpr int buf = decltype(buf_c)::value;
        constexpr int STEPS = D / 8, RPS = 16 / STEPS;  // dP steps, score rows requested per step
        const int qt = q_lo + 32 * t;
        if (t + 1 < ntiles) issue_tile(t + 1, buf ^ 1);
        aim_loads(t + 1);
        const unsigned v_ld = lane_sd + ld_tile, v_st = lane_sd + (unsigned)qt * row_bytes;
        auto request = [&](int step) __attribute__((always_inline)) {
#pragma unroll
            for (int u = 0; u < RPS; ++u) {
                const int r = step * RPS + u;
                s_nx[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs_s, v_ld, row_part[r], 2));
            }
        };
        auto store_ds = [&](int r, float x) __attribute__((always_inline)) {
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, x), rs_ds, v_st, row_part[r], 0);
        };
        if (!wave_hidden(t)) {
            if (!wave_plain(t)) {  // wavefront-uniform, a few tiles per key block
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int qi = qt + 8 * (r >> 2) + 4 * half + (r & 3);
                    const bool hidden = (p.causal && kw > qi) | (qi >= seq_q) | !key_live;
                    s_cur[r] = hidden ? -__builtin_inff() : s_cur[r];
                }
            }
            // ---- dP = dOut_tile . V_blk^T; the fragment of step t8 + 1 is requested before the MFMAs of step t8 ----
            Acc16 dp;
#pragma unroll
            for (int r = 0; r < 16; ++r) dp[r] = 0.f;
            const float *ob = Os + buf * TILE;
            auto frag = [&](int t8) __attribute__((always_inline)) {
                return *reinterpret_cast<const float4 *>(ob + ofrag[t8 & 7] + 4 * ((2 * t8) & 16));
            };
            float4 ov_n = frag(0);
#pragma unroll
            for (int t8 = 0; t8 < STEPS; ++t8) {
                const float4 ov = ov_n;
                if (t8 + 1 < STEPS) ov_n = frag(t8 + 1);
                __builtin_amdgcn_sched_barrier(0);  // the scheduler would otherwise sink the read to just before its use
                dp = __builtin_amdgcn_mfma_f32_32x32x2f32(ov.x, vr[t8].x, dp, 0, 0, 0);
                request(t8);
                dp = __builtin_amdgcn_mfma_f32_32x32x2f32(ov.y, vr[t8].y, dp, 0, 0, 0);
                dp = __builtin_amdgcn_mfma_f32_32x32x2f32(ov.z, vr[t8].z, dp, 0, 0, 0);
                dp = __builtin_amdgcn_mfma_f32_32x32x2f32(ov.w, vr[t8].w, dp, 0, 0, 0);
            }
            // ---- P, dS (lane-local) and the two output products ----
            const float *qb = Qs + buf * TILE + qvec;
            const float *stats = Ls + buf * 128 + 4 * half;
            float4 lse4, del4;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                if ((r & 3) == 0) {
                    lse4 = *reinterpret_cast<const float4 *>(stats + 2 * r);
                    del4 = *reinterpret_cast<const float4 *>(stats + 64 + 2 * r);
                }
                const float pw = __builtin_amdgcn_exp2f(__builtin_fmaf(s_cur[r], c2, -f4_get(lse4, r & 3)));
                const float dsv = pw * (dp[r] - f4_get(del4, r & 3));
                store_ds(r, dsv);
                const VV ov = *reinterpret_cast<const VV *>(ob + ovec[r]);
                const VV qv = *reinterpret_cast<const VV *>(qb + (8 * (r >> 2) + (r & 3)) * D);
#pragma unroll
                for (int e = 0; e < NDT; ++e) {
                    dvT[e] = __builtin_amdgcn_mfma_f32_32x32x2f32(vecn_get(ov, e), pw, dvT[e], 0, 0, 0);
                    dkT[e] = __builtin_amdgcn_mfma_f32_32x32x2f32(vecn_get(qv, e), dsv, dkT[e], 0, 0, 0);
                }
            }
        } else {
            // every (query, key) of this wavefront's part of the tile is masked: dS is zero there
#pragma unroll
            for (int st = 0; st < STEPS; ++st) request(st);
#pragma unroll
            for (int r = 0; r < 16; ++r) store_ds(r, 0.f);
        }
        __builtin_amdgcn_s_waitcnt(0x8F70);  // vmcnt(32)
        __syncthreads();
    };
    for (int t = 0; t < ntiles; t += 2) {
        tile_step(t, std::integral_constant<int, 0>{}, s_a, s_b);
        if (t + 1 < ntiles) tile_step(t + 1, std::integral_constant<int, 1>{}, s_b, s_a);
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
    sdpa_bwd_keys_kernel<D><<<dim3((unsigned)grid), dim3(256), smem, st>>>(a);
    FTH_CHECK_LAUNCH("sdpa_bwd_keys");
    return FTH_OK;
}

// ---------------------------------------------------------------------------------------------
// Query-owned pass: dQ = scale . dS . K. One workgroup per 128 queries (a wavefront owns 32), walking the 32-key tiles
// its queries can see; K tiles through double-buffered LDS (row order, read along d), dS straight from HBM in the
// accumulator layout of the key-owned pass: dQ^T[d, q] += K_tile^T . dS^T, where MFMA step r contracts over the two
// keys 8 (r / 4) + 4 half + r % 4 and a lane's B operand is dS[q = lane % 32][that key] - four 16-byte loads per lane
// and tile, requested one tile ahead. The key-owned pass stored explicit zeros for the masked pairs of every tile on
// the diagonal, so this loop has no mask logic: a wavefront simply stops at the last tile its queries reach. 64 MFMAs
// (D = 128) per tile against 4 loads and 16 LDS reads, and hardly a vector instruction in between.
// ---------------------------------------------------------------------------------------------
struct DqArgs {
    const float *ds, *k;
    float *dq;
    int64_t num_bh;
    int seq_q, seq_k;
    float scale;
    int causal;
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
    const int64_t pid = blockIdx.x;
    const int q_blocks = (p.seq_q + 127) / 128;
    const int qb = q_blocks - 1 - (int)(pid / p.num_bh);  // heaviest (latest) query blocks first under a causal mask
    const int64_t bh = pid % p.num_bh;
    const int seq_q = p.seq_q, seq_k = p.seq_k;
    const int q_blk0 = qb * 128, q_wave0 = q_blk0 + 32 * wave, qi = q_wave0 + lq;
    const bool q_live = qi < seq_q;
    const float *Kg = p.k + bh * (int64_t)seq_k * D;
    const float *DSg = p.ds + bh * (int64_t)seq_q * seq_k;

    int blk_last_q = q_blk0 + 127, wave_last_q = q_wave0 + 31;
    if (blk_last_q > seq_q - 1) blk_last_q = seq_q - 1;
    if (wave_last_q > seq_q - 1) wave_last_q = seq_q - 1;
    int k_end = seq_k;
    if (p.causal && blk_last_q + 1 < k_end) k_end = blk_last_q + 1;
    const int ntiles = (k_end + 31) / 32;

    // ---- K tile loader (rows past the last key clamped: their dS is read as zero) ----
    const unsigned lds0 = __builtin_amdgcn_readfirstlane((unsigned)reinterpret_cast<uintptr_t>(smem_raw));
    const unsigned wave_u = __builtin_amdgcn_readfirstlane((unsigned)wave);
    auto issue_tile = [&](int t, int buf) __attribute__((always_inline)) {
        const unsigned dst = lds0 + (unsigned)(buf * TILE * 4) + wave_u * (CPW * 1024u);
#pragma unroll
        for (int ci = 0; ci < CPW; ++ci) {
            int row = 32 * t + (wave * CPW + ci) * RPC + lane / VPR;
            row = row < seq_k ? row : seq_k - 1;
            load_to_lds_16(Kg, (unsigned)row * (unsigned)(D * 4) + 16u * (unsigned)(lane % VPR), dst + ci * 1024u);
        }
    };

    // ---- dS through range-checked buffer loads: lane part (its query's row, its half's keys) in the vector offset,
    //      tile part in the scalar offset; a dead query's lane part is "nowhere" ----
    constexpr unsigned kOut = 0x40000000u;
    const unsigned row_bytes = (unsigned)seq_k * 4u;
    const __amdgpu_buffer_rsrc_t rs_ds =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(DSg), 0, (int)((unsigned)seq_q * row_bytes), 0x00020000);
    const unsigned lane_ds = q_live ? (unsigned)qi * row_bytes + 16u * (unsigned)half : kOut;
    typedef unsigned u4v __attribute__((ext_vector_type(4)));
    auto wave_active = [&](int t) __attribute__((always_inline)) { return !p.causal || 32 * t <= wave_last_q; };
    auto load_ds = [&](int t, float4(&dst)[4]) __attribute__((always_inline)) {
        const bool none = t >= ntiles || !wave_active(t);
        const unsigned v = none ? kOut : lane_ds;
        const bool tail = 32 * t + 32 > seq_k;  // uniform: the last keys of a row must not run into the next row
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            u4v x = __builtin_amdgcn_raw_buffer_load_b128(rs_ds, v, (unsigned)(32 * t + 8 * g) * 4u, 2);
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
            const float *kb = Ks + buf * TILE + kvec;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const VV kv = *reinterpret_cast<const VV *>(kb + (8 * (r >> 2) + (r & 3)) * D);
                const float w = f4_get(ds_cur[r >> 2], r & 3);
#pragma unroll
                for (int e = 0; e < NDT; ++e) acc[e] = __builtin_amdgcn_mfma_f32_32x32x2f32(vecn_get(kv, e), w, acc[e], 0, 0, 0);
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
    sdpa_bwd_dq_kernel<D><<<dim3((unsigned)grid), dim3(256), smem, st>>>(a);
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
    return !off && d_k == d_v && (d_k == 64 || d_k == 128) && seq_q % 4 == 0 && seq_k % 4 == 0 && seq_q >= 32 && seq_k >= 32 &&
           scale > 0.f && (seq_q + 64) * seq_k < ((int64_t)1 << 28) && seq_q * d_k < (1 << 28);  // byte offsets inside one slab of S stay below 2^30
}

int32_t sdpa_backward_keys_f32(const float *q, const float *v, const float *dout, int64_t dout_bh_stride, const float *s, const float *lse,
                               const float *delta, int64_t num_bh, int64_t seq_q, int64_t seq_k, int64_t d, float scale, int causal,
                               int64_t row_block, float *ds, float *dk, float *dv, hipStream_t st) {
    KeysArgs a;
    a.q = q; a.v = v; a.dout = dout; a.s = s; a.lse = lse; a.delta = delta;
    a.ds = ds; a.dk = dk; a.dv = dv;
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
