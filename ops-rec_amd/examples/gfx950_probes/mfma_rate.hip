// Probe: rate of the two bf16 matrix instructions of gfx950 the forward kernels use, v_mfma_f32_32x32x16_bf16 (persistent
// kernel, 32 query rows per wavefront) and v_mfma_f32_16x16x32_bf16 (kernel for short lists, 16 rows), with one, two
// and four wavefronts per SIMD issuing four independent accumulators each.
//   hipcc --offload-arch=gfx950 -O3 -o /tmp/mfma_rate mfma_rate.hip && /tmp/mfma_rate
#include <hip/hip_runtime.h>
#include <stdio.h>
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f4;
typedef __attribute__((ext_vector_type(16))) float f16v;
template <int MODE>
__global__ __launch_bounds__(256) void k(float* out, int iters) {
    bf16x8 a, b;
    for (int i = 0; i < 8; ++i) { a[i] = (__bf16)(threadIdx.x * 0.001f + i); b[i] = (__bf16)(i * 0.5f); }
    if (MODE == 0) {
        f4 c0 = {0,0,0,0}, c1 = c0, c2 = c0, c3 = c0;
        for (int it = 0; it < iters; ++it) {
            c0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c1, 0, 0, 0);
            c2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c2, 0, 0, 0);
            c3 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c3, 0, 0, 0);
        }
        out[blockIdx.x * 256 + threadIdx.x] = c0[0] + c1[1] + c2[2] + c3[3];
    } else {
        f16v c0, c1, c2, c3;
        for (int i = 0; i < 16; ++i) { c0[i] = 0; c1[i] = 0; c2[i] = 0; c3[i] = 0; }
        for (int it = 0; it < iters; ++it) {
            c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
            c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c2, 0, 0, 0);
            c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c3, 0, 0, 0);
        }
        out[blockIdx.x * 256 + threadIdx.x] = c0[0] + c1[1] + c2[2] + c3[3];
    }
}
int main() {
    float* out; hipMalloc(&out, 1024 * 256 * 4);
    hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
    const int iters = 20000;
    for (int mode = 0; mode < 2; ++mode) for (int wg = 256; wg <= 1024; wg *= 2) {
        for (int rep = 0; rep < 2; ++rep) {
            hipEventRecord(e0);
            if (mode == 0) hipLaunchKernelGGL(k<0>, dim3(wg), dim3(256), 0, 0, out, iters);
            else hipLaunchKernelGGL(k<1>, dim3(wg), dim3(256), 0, 0, out, iters);
            hipEventRecord(e1); hipEventSynchronize(e1);
            float ms; hipEventElapsedTime(&ms, e0, e1);
            if (rep == 1) {
                double mfmas_per_simd = (double)iters * 4 * (wg / 256.0);  // waves per SIMD = wg/256 (4 waves per wg, 1024 SIMDs)
                double flop = (double)iters * 4 * wg * 4 * 2.0 * (mode == 0 ? 16*16*32 : 32*32*16);
                printf("%s workgroups %d: %.3f ms, %.1f ns per MFMA per SIMD, %.1f TFLOP/s\n", mode == 0 ? "16x16x32" : "32x32x16", wg, ms, ms * 1e6 / mfmas_per_simd, flop / ms / 1e9);
            }
        }
    }
    return 0;
}
