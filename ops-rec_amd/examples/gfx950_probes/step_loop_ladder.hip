// Probe: the time step of the persistent forward kernel in isolation (no global memory): the 16 MFMAs of a 32-key
// sub-tile, its SiLU, the LDS operand reads and the barrier, added one at a time, in several workgroup shapes.
//   hipcc --offload-arch=gfx950 -O3 -o /tmp/step_loop_ladder step_loop_ladder.hip && /tmp/step_loop_ladder
// step-loop probe: MFMA + SiLU + LDS operand reads (+ barrier) in the forward kernel's instruction mix
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdint>
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(4))) short short4_t;
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s at %d\n", hipGetErrorString(e), __LINE__); return 1;} } while (0)
__device__ __forceinline__ u32x2 tr(const uint16_t* p) {
  typedef short4_t __attribute__((address_space(3))) * lp;
  return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lp)p));
}
__device__ __forceinline__ uint32_t pk2(float a, float b) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2; bf16x2 r; r[0] = (__bf16)a; r[1] = (__bf16)b; return __builtin_bit_cast(uint32_t, r);
}
// WPB waves per block, BPC blocks per CU, RW 32-row blocks per wave, READS 0 none 1 both 2 K only 3 V only,
// LOOK operand lookahead, BAR barrier per step, SILU 0 none 1 full
template <int WPB, int BPC, int RW, int READS, int LOOK, bool BAR, int SILU>
__global__ __launch_bounds__(WPB * 64) __attribute__((amdgpu_waves_per_eu((WPB * BPC) / 4, (WPB * BPC) / 4)))
void k(float* out, unsigned long long* clk, int iters, float c_exp) {
  constexpr int THREADS = WPB * 64;
  __shared__ __attribute__((aligned(16))) uint16_t lk[4096 * 4];
  __shared__ __attribute__((aligned(16))) uint16_t lv[4096 * 4];
  __shared__ uint16_t pad[BPC == 1 ? 30000 : 4000];  // occupancy control through LDS
  int tid = threadIdx.x, lane = tid & 63;
  for (int i = tid; i < 16384; i += THREADS) { lk[i] = i; lv[i] = i * 3; }
  pad[tid] = tid;
  __syncthreads();
  f32x16 s_a[RW], s_b[RW], o[RW][4];
  for (int r = 0; r < RW; ++r) for (int i = 0; i < 16; ++i) { s_a[r][i] = tid * 0.01f + i * 0.1f + r; s_b[r][i] = s_a[r][i] + 1; for (int m = 0; m < 4; ++m) o[r][m][i] = 0; }
  u32x4 q[RW][8]; for (int r = 0; r < RW; ++r) for (int j = 0; j < 8; ++j) q[r][j] = u32x4{(uint32_t)j, 2, 3, (uint32_t)r};
  uint32_t pa[RW][8], pb[RW][8]; for (int r = 0; r < RW; ++r) for (int i = 0; i < 8; ++i) { pa[r][i] = i; pb[r][i] = i + 1; }
  const int koff = (lane & 31) * 128 + (((lane >> 5)) ^ (lane & 15)) * 8;
  const int voff = ((lane >> 5) * 4 + ((lane & 15) >> 2)) * 128 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  auto pair = [&](const f32x16& s, int i, uint32_t* pk) {
    if (SILU == 0) { pk[i] ^= 1; return; }
    float t0 = s[2 * i] * c_exp, t1 = s[2 * i + 1] * c_exp;
    t0 = __builtin_amdgcn_exp2f(t0); t1 = __builtin_amdgcn_exp2f(t1);
    t0 = 1.0f + t0; t1 = 1.0f + t1;
    t0 = __builtin_amdgcn_rcpf(t0); t1 = __builtin_amdgcn_rcpf(t1);
    pk[i] = pk2(s[2 * i] * t0, s[2 * i + 1] * t1);
  };
  auto rk = [&](int it, int c) -> u32x4 {
    if (READS == 1 || READS == 2) return *reinterpret_cast<const u32x4*>(&lk[(koff ^ (c * 16)) + (it & 3) * 4096]);
    return u32x4{1, 2, 3, (uint32_t)c};
  };
  auto rv = [&](int it, int c) -> u32x4 {
    if (READS == 1 || READS == 3) { const uint16_t* p = &lv[voff + (c & 3) * 32 + (c >> 2) * 2048 + (it & 3) * 4096]; u32x2 lo = tr(p), hi = tr(p + 1024); return u32x4{lo[0], lo[1], hi[0], hi[1]}; }
    return u32x4{5, 6, 7, (uint32_t)c};
  };
  unsigned long long t0 = __builtin_amdgcn_s_memtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int par = 0; par < 2; ++par) {
      f32x16* s_cur = par ? s_b : s_a; f32x16* s_nxt = par ? s_a : s_b;
      uint32_t (*pk_cur)[8] = par ? pb : pa; uint32_t (*pk_prev)[8] = par ? pa : pb;
      u32x4 vop[8];
#pragma unroll
      for (int c = 0; c < LOOK; ++c) vop[c] = rv(it, c);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int c = 0; c < 8; ++c) {
#pragma unroll
        for (int r = 0; r < RW; ++r) {
          u32x4 p4 = {pk_prev[r][4 * (c / 4)], pk_prev[r][4 * (c / 4) + 1], pk_prev[r][4 * (c / 4) + 2], pk_prev[r][4 * (c / 4) + 3]};
          o[r][c & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vop[c]), __builtin_bit_cast(bf16x8, p4), o[r][c & 3], 0, 0, 0);
        }
        if (c + LOOK < 8) vop[c + LOOK] = rv(it, c + LOOK);
        if (RW == 2) pair(s_cur[c & 1], c / 2, pk_cur[c & 1]); else if (!(c & 1)) pair(s_cur[0], c / 2, pk_cur[0]);
        __builtin_amdgcn_sched_barrier(0);
      }
      u32x4 kop[8];
#pragma unroll
      for (int c = 0; c < LOOK; ++c) kop[c] = rk(it, c);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int c = 0; c < 8; ++c) {
#pragma unroll
        for (int r = 0; r < RW; ++r) {
          f32x16 z; for (int i = 0; i < 16; ++i) z[i] = 0;
          s_nxt[r] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kop[c]), __builtin_bit_cast(bf16x8, q[r][c]), c == 0 ? z : s_nxt[r], 0, 0, 0);
        }
        if (c + LOOK < 8) kop[c + LOOK] = rk(it, c + LOOK);
        if (RW == 2) pair(s_cur[c & 1], 4 + c / 2, pk_cur[c & 1]); else if (!(c & 1)) pair(s_cur[0], 4 + c / 2, pk_cur[0]);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (BAR) { __builtin_amdgcn_sched_barrier(0); __builtin_amdgcn_s_barrier(); __builtin_amdgcn_sched_barrier(0); }
    }
  }
  unsigned long long t1 = __builtin_amdgcn_s_memtime();
  if (blockIdx.x == 0 && tid == 0) clk[0] = t1 - t0;
  float r = 0; for (int w = 0; w < RW; ++w) { for (int m = 0; m < 4; ++m) for (int i = 0; i < 16; ++i) r += o[w][m][i]; for (int i = 0; i < 8; ++i) r += pa[w][i] + pb[w][i]; r += s_a[w][0] + s_b[w][1]; }
  out[blockIdx.x * THREADS + tid] = r + pad[5];
}
template <int WPB, int BPC, int RW, int READS, int LOOK, bool BAR, int SILU> int run(const char* note) {
  float* out; CK(hipMalloc(&out, 2048 * 512 * 4));
  unsigned long long* clk; CK(hipMalloc(&clk, 64)); CK(hipMemset(clk, 0, 64));
  int iters = 1500; int blocks = 256 * BPC;
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  k<WPB, BPC, RW, READS, LOOK, BAR, SILU><<<blocks, WPB * 64>>>(out, clk, 30, -0.1f); CK(hipDeviceSynchronize());
  CK(hipEventRecord(e0)); k<WPB, BPC, RW, READS, LOOK, BAR, SILU><<<blocks, WPB * 64>>>(out, clk, iters, -0.1f); CK(hipEventRecord(e1)); CK(hipDeviceSynchronize());
  float ms; CK(hipEventElapsedTime(&ms, e0, e1));
  unsigned long long cyc = 0; CK(hipMemcpy(&cyc, clk, 8, hipMemcpyDeviceToHost));
  double subtiles_per_simd = (double)BPC * WPB * RW / 4.0;
  double ns = ms * 1e6 / (iters * 2) / subtiles_per_simd;
  double cyc_per = (double)cyc / (iters * 2) / subtiles_per_simd;
  printf("wpb=%d bpc=%d rw=%d reads=%d look=%d bar=%d silu=%d : %4.0f ns, %5.0f clk per sub-tile per SIMD (%.2f GHz)  %s\n", WPB, BPC, RW, READS, LOOK, (int)BAR, SILU, ns, cyc_per, cyc_per / ns, note);
  fflush(stdout);
  CK(hipFree(out)); CK(hipFree(clk)); return 0;
}
int main() {
  run<4, 2, 1, 0, 2, false, 1>("floor: no LDS reads");
  run<4, 2, 1, 1, 2, false, 1>("LDS reads");
  run<4, 2, 1, 1, 2, true, 1>("LDS reads + barrier (the persistent kernel's shape)");
  run<8, 1, 1, 1, 2, true, 1>("8-wave block");
  run<8, 1, 1, 1, 2, false, 1>("8-wave block, no barrier");
  run<4, 2, 1, 2, 2, false, 1>("K reads only");
  run<4, 2, 1, 3, 2, false, 1>("V reads only");
  run<4, 2, 1, 1, 4, true, 1>("lookahead 4");
  run<4, 2, 1, 1, 8, true, 1>("lookahead 8");
  run<4, 2, 1, 1, 2, false, 0>("no silu, LDS reads");
  run<4, 2, 1, 0, 2, false, 0>("no silu, no reads (pure MFMA)");
  run<4, 1, 1, 0, 2, false, 1>("one wave per SIMD, 32 rows, no reads");
  run<4, 1, 1, 1, 2, false, 1>("one wave per SIMD, 32 rows, reads");
  run<4, 1, 2, 0, 2, false, 1>("one wave per SIMD, 64 rows, no reads");
  run<4, 1, 2, 1, 2, false, 1>("one wave per SIMD, 64 rows, reads");
  run<4, 1, 2, 1, 2, true, 1>("one wave per SIMD, 64 rows, reads, barrier");
  run<4, 1, 2, 1, 4, true, 1>("one wave per SIMD, 64 rows, reads, barrier, look 4");
  run<4, 1, 2, 1, 2, false, 0>("one wave per SIMD, 64 rows, reads, no silu");
  return 0;
}
