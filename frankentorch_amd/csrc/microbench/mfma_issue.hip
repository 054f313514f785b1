// Microbenchmark behind the design rule of the MFMA kernels: which instruction classes overlap with MFMAs on gfx950?
// A register-only loop of four independent accumulators, 256 workgroups of four wavefronts (one per SIMD; 512
// workgroups = two per SIMD), with NF filler instructions after every MFMA. Prints cycles per MFMA slot at 2.4 GHz.
// KIND: 0 v_mfma_f32_32x32x2_f32, 1 v_mfma_i32_32x32x32_i8, 2 v_mfma_f64_16x16x4_f64.
// FILL: 0 none, 1 fp32 FMA, 2 LDS read, 3 SALU, 4 v_exp_f32, 5 integer VALU (two instructions per unit), 6 global load.
// Build: hipcc -O3 --offload-arch=gfx950 -o microbench_mfma_issue mfma_issue.hip (frankentorch_amd/build.py does it).
#include <hip/hip_runtime.h>
#include <cstdio>
using F16v = float __attribute__((ext_vector_type(16)));
using I16v = int __attribute__((ext_vector_type(16)));
using I4v = int __attribute__((ext_vector_type(4)));
using D4v = double __attribute__((ext_vector_type(4)));
template <int KIND, int FILL, int NF>
__global__ __launch_bounds__(256) void k(float *out, const float *gin, int iters, float a0, int s0) {
    extern __shared__ float sm[];
    F16v fa[4]; I16v ia[4]; D4v da[4];
    for (int i = 0; i < 4; ++i) { for (int r = 0; r < 16; ++r) { fa[i][r] = 0.f; ia[i][r] = 0; } for (int r = 0; r < 4; ++r) da[i][r] = 0.0; }
    float a = a0 + threadIdx.x, b = a0 * 2.f, x = a0; int xi = threadIdx.x; int sx = s0;
    I4v av = {xi, xi + 1, xi + 2, xi + 3}, bv = {1, 2, 3, 4};
    double ad = a, bd = b;
    float4 lacc = make_float4(0, 0, 0, 0);
    sm[threadIdx.x] = a;
    __syncthreads();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (KIND == 0) fa[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, fa[i], 0, 0, 0);
                if (KIND == 1) ia[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bv, ia[i], 0, 0, 0);
                if (KIND == 2) da[i] = __builtin_amdgcn_mfma_f64_16x16x4f64(ad, bd, da[i], 0, 0, 0);
#pragma unroll
                for (int v = 0; v < NF; ++v) {
                    if (FILL == 1) x = __builtin_fmaf(x, 1.0001f, 0.5f);
                    if (FILL == 2) { float4 t = *reinterpret_cast<const float4 *>(sm + ((threadIdx.x * 4 + 64 * (u + v)) & 1023)); lacc.x += t.x; }
                    if (FILL == 3) { sx = sx * 3 + 1; }
                    if (FILL == 4) x = __builtin_amdgcn_exp2f(x);
                    if (FILL == 5) xi = xi + (xi >> 3);
                    if (FILL == 6) { lacc.y += gin[(threadIdx.x + 64 * (u * 4 + i + v) + xi * 0) & 4095]; }
                }
            }
        }
    }
    float s = x + xi + lacc.x + lacc.y + sx;
    for (int i = 0; i < 4; ++i) { for (int r = 0; r < 16; ++r) s += fa[i][r] + ia[i][r]; for (int r = 0; r < 4; ++r) s += (float)da[i][r]; }
    out[blockIdx.x * 256 + threadIdx.x] = s;
}
float *g_out, *g_in;

// ---- second part: does the sustained MFMA rate depend on the operand VALUES? Register-only, no memory: the operands come from
//      four register sets filled with zeros, ones or hashed bits. ----
__device__ unsigned hash32(unsigned x) { x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16; return x; }
template <int KIND>
__global__ __launch_bounds__(256) void kd(float *out, int iters, int mode) {
    F16v fa[4]; I16v ia[4];
    for (int i = 0; i < 4; ++i) for (int r = 0; r < 16; ++r) { fa[i][r] = 0.f; ia[i][r] = 0; }
    I4v av[4], bv[4]; float af[4], bf[4];
    for (int s = 0; s < 4; ++s) {
        for (int e = 0; e < 4; ++e) {
            unsigned h = hash32(threadIdx.x * 131 + s * 17 + e * 7 + blockIdx.x * 977), g = hash32(h + 12345);
            if (mode == 0) { h = 0; g = 0; }
            if (mode == 1) { h = 0x01010101u; g = 0x01010101u; }
            av[s][e] = (int)h; bv[s][e] = (int)g;
        }
        const unsigned h = hash32(threadIdx.x * 31 + s);
        af[s] = mode == 0 ? 0.f : mode == 1 ? 1.f : (float)(int)(h & 0xffff) / 65536.f - 0.5f;
        bf[s] = mode == 0 ? 0.f : mode == 1 ? 1.f : (float)(int)((h >> 16) & 0xffff) / 65536.f - 0.5f;
    }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (KIND == 0) fa[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[(u + i) & 3], bf[(u + 2 * i) & 3], fa[i], 0, 0, 0);
                if (KIND == 1) ia[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[(u + i) & 3], bv[(u + 2 * i) & 3], ia[i], 0, 0, 0);
            }
        }
    }
    float s = 0;
    for (int i = 0; i < 4; ++i) for (int r = 0; r < 16; ++r) s += fa[i][r] + ia[i][r];
    out[blockIdx.x * 256 + threadIdx.x] = s;
}
template <int KIND> void run_data(const char *name, int mode) {
    const int iters = 20000;
    hipEvent_t e0, e1; (void)hipEventCreate(&e0); (void)hipEventCreate(&e1);
    kd<KIND><<<256, 256>>>(g_out, 100, mode);
    (void)hipEventRecord(e0);
    kd<KIND><<<256, 256>>>(g_out, iters, mode);
    (void)hipEventRecord(e1); (void)hipEventSynchronize(e1);
    float ms; (void)hipEventElapsedTime(&ms, e0, e1);
    const double n = (double)iters * 32 * 1024, ops = KIND == 1 ? n * 65536 : n * 4096;
    printf("%-44s %7.2f ms  %8.3f %s\n", name, ms, ops / (ms * 1e-3) / (KIND == 1 ? 1e15 : 1e12), KIND == 1 ? "POP/s" : "TFLOP/s");
}
template <int KIND, int FILL, int NF> void run(const char *name, int blocks) {
    int smem = blocks == 256 ? 100 * 1024 : 60 * 1024;
    int iters = 1000;
    hipEvent_t e0, e1; (void)hipEventCreate(&e0); (void)hipEventCreate(&e1);
    (void)hipFuncSetAttribute((const void *)k<KIND, FILL, NF>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    k<KIND, FILL, NF><<<blocks, 256, smem>>>(g_out, g_in, 10, 1.f, 3);
    (void)hipEventRecord(e0);
    k<KIND, FILL, NF><<<blocks, 256, smem>>>(g_out, g_in, iters, 1.f, 3);
    (void)hipEventRecord(e1); (void)hipEventSynchronize(e1);
    float ms; (void)hipEventElapsedTime(&ms, e0, e1);
    double per = ms * 1e6 / ((double)iters * 32 * (blocks / 256.0)) * 2.4;
    printf("%-44s w/SIMD %d: %6.1f cycles per MFMA slot\n", name, blocks / 256, per);
}
int main() {
    (void)hipMalloc(&g_out, 4 * 256 * 1024); (void)hipMalloc(&g_in, 4 * 4096); (void)hipMemset(g_in, 0, 4 * 4096);
    run<0, 0, 0>("f32 32x32x2 alone", 256);
    run<0, 1, 4>("f32 + 4 VALU fma", 256);
    run<0, 5, 4>("f32 + 4 VALU int", 256);
    run<0, 4, 2>("f32 + 2 v_exp", 256);
    run<0, 2, 2>("f32 + 2 ds_read_b128", 256);
    run<0, 3, 4>("f32 + 4 SALU", 256);
    run<0, 6, 2>("f32 + 2 global_load", 256);
    run<0, 1, 4>("f32 + 4 VALU fma", 512);
    run<0, 2, 2>("f32 + 2 ds_read_b128", 512);
    run<1, 0, 0>("i8 32x32x32 alone", 256);
    run<1, 1, 4>("i8 + 4 VALU fma", 256);
    run<1, 5, 4>("i8 + 4 VALU int", 256);
    run<1, 2, 2>("i8 + 2 ds_read_b128", 256);
    run<1, 1, 4>("i8 + 4 VALU fma", 512);
    run<2, 0, 0>("f64 16x16x4 alone", 256);
    run<2, 1, 4>("f64 + 4 VALU fma", 256);
    run<2, 2, 2>("f64 + 2 ds_read_b128", 256);
    run<2, 1, 4>("f64 + 4 VALU fma", 512);
    printf("operand values, register-only loops (no memory traffic):\n");
    run_data<1>("i8 32x32x32, all-zero operands", 0);
    run_data<1>("i8 32x32x32, all-one bytes", 1);
    run_data<1>("i8 32x32x32, random bytes", 2);
    run_data<0>("f32 32x32x2, all-zero operands", 0);
    run_data<0>("f32 32x32x2, ones", 1);
    run_data<0>("f32 32x32x2, random in [-0.5, 0.5)", 2);
    return 0;
}
