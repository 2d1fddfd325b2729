// Probe: issue rate of the vector instructions of the SiLU epilogue on gfx950, per wavefront and per SIMD, with two
// and eight wavefronts per SIMD: plain (v_mul_f32), transcendental (v_exp_f32), and the two mixed in one stream.
//   hipcc --offload-arch=gfx950 -O3 -o /tmp/instruction_rates instruction_rates.hip && /tmp/instruction_rates
#include <hip/hip_runtime.h>
#include <cstdio>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s at %d\n", hipGetErrorString(e), __LINE__); return 1;} } while (0)
#define REP8(op) op(0) op(1) op(2) op(3) op(4) op(5) op(6) op(7)
#define KERNEL(name, ASM)                                                                     \
  __global__ __launch_bounds__(256) void name(float* out, int iters, unsigned long long* cyc) { \
    float x0 = threadIdx.x * 0.001f + 1, x1 = x0 + 1, x2 = x0 + 2, x3 = x0 + 3, x4 = x0 + 4, x5 = x0 + 5, x6 = x0 + 6, x7 = x0 + 7; \
    unsigned long long t0 = __builtin_amdgcn_s_memtime();                                     \
    for (int it = 0; it < iters; ++it) {                                                      \
      asm volatile(ASM("%0") ASM("%1") ASM("%2") ASM("%3") ASM("%4") ASM("%5") ASM("%6") ASM("%7")  \
                   ASM("%0") ASM("%1") ASM("%2") ASM("%3") ASM("%4") ASM("%5") ASM("%6") ASM("%7")  \
                   : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3), "+v"(x4), "+v"(x5), "+v"(x6), "+v"(x7)); \
    }                                                                                         \
    unsigned long long t1 = __builtin_amdgcn_s_memtime();                                     \
    out[blockIdx.x * 256 + threadIdx.x] = x0 + x1 + x2 + x3 + x4 + x5 + x6 + x7;              \
    if (threadIdx.x == 0 && blockIdx.x == 0) *cyc = t1 - t0;                                  \
  }
#define A_EXP32(r) "v_exp_f32 " r ", " r "\n"
#define A_RCP32(r) "v_rcp_f32 " r ", " r "\n"
#define A_EXP16(r) "v_exp_f16 " r ", " r "\n"
#define A_RCP16(r) "v_rcp_f16 " r ", " r "\n"
#define A_MUL32(r) "v_mul_f32 " r ", " r ", " r "\n"
#define A_PKMUL16(r) "v_pk_mul_f16 " r ", " r ", " r "\n"
#define A_PKADD16(r) "v_pk_add_f16 " r ", " r ", " r "\n"
#define A_CVTBF(r) "v_cvt_pk_bf16_f32 " r ", " r ", " r "\n"
#define A_CVTRTZ(r) "v_cvt_pkrtz_f16_f32 " r ", " r ", " r "\n"
#define A_EXP16S(r) "v_exp_f16_sdwa " r ", " r " dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_1\n"
#define A_RCP16S(r) "v_rcp_f16_sdwa " r ", " r " dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_1\n"
#define A_SQRT(r) "v_rsq_f32 " r ", " r "\n"
#define A_CVT16_32(r) "v_cvt_f32_f16 " r ", " r "\n"
#define A_MIX(r) "v_exp_f32 " r ", " r "\nv_mul_f32 " r ", " r ", " r "\n"
#define A_MIX3(r) "v_exp_f32 " r ", " r "\nv_mul_f32 " r ", " r ", " r "\nv_add_f32 " r ", " r ", " r "\nv_mul_f32 " r ", " r ", " r "\n"
KERNEL(k_mix, A_MIX) KERNEL(k_mix3, A_MIX3)
KERNEL(k_exp32, A_EXP32) KERNEL(k_rcp32, A_RCP32) KERNEL(k_exp16, A_EXP16) KERNEL(k_rcp16, A_RCP16) KERNEL(k_mul32, A_MUL32)
KERNEL(k_pkmul16, A_PKMUL16) KERNEL(k_pkadd16, A_PKADD16) KERNEL(k_cvtbf, A_CVTBF) KERNEL(k_cvtrtz, A_CVTRTZ)
KERNEL(k_exp16s, A_EXP16S) KERNEL(k_rcp16s, A_RCP16S) KERNEL(k_rsq, A_SQRT) KERNEL(k_cvt1632, A_CVT16_32)
template <typename K> int run(K kern, const char* name, int wps) {
  float* out; unsigned long long* cyc; CK(hipMalloc(&out, 4096 * 256 * 4)); CK(hipMalloc(&cyc, 8));
  int iters = 20000;
  kern<<<256 * wps, 256>>>(out, 100, cyc); CK(hipDeviceSynchronize());
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  CK(hipEventRecord(e0)); kern<<<256 * wps, 256>>>(out, iters, cyc); CK(hipEventRecord(e1)); CK(hipDeviceSynchronize());
  float ms; CK(hipEventElapsedTime(&ms, e0, e1));
  unsigned long long c; CK(hipMemcpy(&c, cyc, 8, hipMemcpyDeviceToHost));
  printf("%-22s waves/SIMD=%d : one wave issues every %.2f cycles; SIMD throughput %.2f ns per instruction (%.2f cycles at 2.4 GHz)\n", name, wps, (double)c / iters / 16, ms * 1e6 / ((double)iters * 16 * wps), ms * 1e6 / ((double)iters * 16 * wps) * 2.4);
  hipFree(out); hipFree(cyc); return 0;
}
int main() {
  for (int w : {2, 8}) {
    run(k_mul32, "v_mul_f32", w); run(k_exp32, "v_exp_f32", w); run(k_rcp32, "v_rcp_f32", w);
    run(k_cvtbf, "v_cvt_pk_bf16_f32", w); run(k_exp16, "v_exp_f16", w); run(k_rcp16, "v_rcp_f16", w);
    run(k_pkmul16, "v_pk_mul_f16", w);
    run(k_mix, "exp+mul (2 instr)", w); run(k_mix3, "exp+mul+add+mul (4 instr)", w);
  }
  return 0;
}
