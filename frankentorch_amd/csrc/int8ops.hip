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
// Product kernel: v_mfma_i32_32x32x32_i8, 128 x 128 output tile per workgroup (2 x 2 wavefronts of
// 64 x 64), K in steps of 64 bytes through double-buffered LDS filled by global_load_lds_dwordx4. Both
// operands are k-contiguous ([m, k] activations, [n, k] weights), so a lane's fragment is 16 consecutive
// bytes of one row. Rows are 64 bytes in LDS; 16-byte slot q of row r is stored at q ^ ((r >> 2) & 3),
// which spreads any 16 consecutive rows of one slot over all 64 banks. Rows past m / n are clamped to the
// last valid row on the load side and never stored. Shapes whose K is not a multiple of 64 or whose
// operands are not 16-byte aligned take a plain one-thread-per-output kernel.

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

// ---- the product -------------------------------------------------------------------------------------
struct I8Args {
    const int8_t *a;  // [m, k] quantised activations
    const int8_t *b;  // [n, k] quantised weights
    const float *a_scales, *b_scales, *bias;
    float *c;  // [m, n]
    int64_t m, n, k;
    int tiles_m, tiles_n;
};

__device__ __forceinline__ void load_to_lds_16(const int8_t *src, unsigned lds_chunk) {
    // Inline assembly so that the compiler's wait-count insertion does not see an LDS write it cannot
    // disambiguate; the kernel waits for vmcnt(0) itself before each barrier.
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(__builtin_amdgcn_readfirstlane(lds_chunk))
                 : "memory", "m0");
}

constexpr int kBM = 128, kBN = 128, kBK = 64;  // bytes of K per stage
constexpr int kTileBytes = kBM * kBK;          // 8 KiB per operand per stage

__global__ __launch_bounds__(256, 2) void i8_gemm_kernel(const I8Args p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];  // [2][A 8 KiB | B 8 KiB]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;  // 2 x 2 wavefronts
    // tiles walked so that the 8 workgroups of consecutive ids (one per XCD, round-robin) share tile rows
    const int tile = blockIdx.x;
    const int tile_m = tile / p.tiles_n, tile_n = tile % p.tiles_n;
    const int64_t m0 = (int64_t)tile_m * kBM, n0 = (int64_t)tile_n * kBN;

    // Loader: one wavefront instruction covers 16 rows x 64 bytes; a wavefront loads 32 rows of A and 32 of B
    // per stage (2 + 2 instructions). Lane L -> row L / 4 of the 16, slot L % 4, fetched from the
    // swizzled source slot so that the LDS image is already swizzled.
    const unsigned lds0 = __builtin_amdgcn_readfirstlane((unsigned)reinterpret_cast<uintptr_t>(smem));
    const unsigned wave_u = __builtin_amdgcn_readfirstlane((unsigned)wave);
    const int lrow = lane >> 2, lslot = lane & 3;
    const int8_t *a_src[2], *b_src[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int r = wave * 32 + i * 16 + lrow;  // row inside the tile
        const int q = lslot ^ ((r >> 2) & 3);     // the logical slot that lives at physical slot lslot
        int64_t ar = m0 + r, br = n0 + r;
        ar = ar < p.m ? ar : p.m - 1;
        br = br < p.n ? br : p.n - 1;
        a_src[i] = p.a + ar * p.k + q * 16;
        b_src[i] = p.b + br * p.k + q * 16;
    }
    auto issue = [&](int kt, int buf) __attribute__((always_inline)) {
        const unsigned base = lds0 + (unsigned)buf * (2 * kTileBytes) + wave_u * 2048u;
        const int64_t koff = (int64_t)kt * kBK;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            load_to_lds_16(a_src[i] + koff, base + i * 1024u);
            load_to_lds_16(b_src[i] + koff, base + kTileBytes + i * 1024u);
        }
    };

    V16i acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    const int num_kt = (int)(p.k / kBK);
    issue(0, 0);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();
    // Fragment addresses: lane (row = lane % 32 of a 32-row MFMA tile, k group = lane / 32).
    const int frow = lane & 31, kg = lane >> 5;
    for (int kt = 0; kt < num_kt; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < num_kt) issue(kt + 1, buf ^ 1);
        const unsigned char *As = smem + buf * (2 * kTileBytes), *Bs = As + kTileBytes;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {  // two 32-byte K steps per stage
            const int q = ks * 2 + kg;
            V4i af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int ra = wm * 64 + i * 32 + frow, rb = wn * 64 + i * 32 + frow;
                af[i] = *reinterpret_cast<const V4i *>(As + ra * kBK + ((q ^ ((ra >> 2) & 3)) << 4));
                bf[i] = *reinterpret_cast<const V4i *>(Bs + rb * kBK + ((q ^ ((rb >> 2) & 3)) << 4));
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
    }

    // Dequantise and store: lane owns column n = lane % 32 of each MFMA tile, rows 8 (r / 4) + 4 (lane / 32) + r % 4.
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int64_t col = n0 + wn * 64 + j * 32 + frow;
        if (col >= p.n) continue;
        const float ws = p.b_scales[col];
        const float bv = p.bias ? p.bias[col] : 0.0f;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t row = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * kg + (r & 3);
                if (row < p.m) {
                    float y = (float)acc[i][j][r] * p.a_scales[row] * ws;
                    if (p.bias) y += bv;
                    p.c[row * p.n + col] = y;
                }
            }
        }
    }
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
    quantize_rows_kernel<<<dim3((unsigned)rows), dim3(256), 0, fth::resolve_stream(s)>>>(x, cols, q, scales);
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
    p.tiles_m = (int)fth::ceil_div(m, kBM);
    p.tiles_n = (int)fth::ceil_div(n, kBN);
    const bool aligned = ((reinterpret_cast<uintptr_t>(x_i8) | reinterpret_cast<uintptr_t>(w_i8)) & 15u) == 0;
    const int64_t tiles = fth::ceil_div(m, kBM) * fth::ceil_div(n, kBN);
    if (k >= kBK && k % kBK == 0 && aligned && tiles <= 2147483647LL) {
        constexpr size_t smem = 2 * 2 * kTileBytes;
        i8_gemm_kernel<<<dim3((unsigned)tiles), dim3(256), smem, st>>>(p);
        FTH_CHECK_LAUNCH("i8_gemm");
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
