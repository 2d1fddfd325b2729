// Probe: variants of the persistent forward kernel's time step in isolation (no global memory): accumulate order,
// SiLU interleave depth, phase separation, operand lookahead, 64-row wavefronts, with a clock calibration.
//   hipcc --offload-arch=gfx950 -O3 -o /tmp/step_loop_variants step_loop_variants.hip && /tmp/step_loop_variants
// step-loop probe 2: accumulate order, SiLU interleave depth, clock calibration
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
// clock calibration: one wave per block, N dependent adds
__global__ void calib(unsigned long long* o, int n, float x) {
  unsigned long long c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  float a = x;
  for (int i = 0; i < n; ++i) {
#pragma unroll
    for (int u = 0; u < 64; ++u) { asm volatile("v_add_f32 %0, %0, %1" : "+v"(a) : "v"(x)); }
  }
  unsigned long long c1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
  if (threadIdx.x == 0) { o[blockIdx.x * 4 + 0] = c1 - c0; o[blockIdx.x * 4 + 1] = r1 - r0; o[blockIdx.x * 4 + 2] = (unsigned long long)a; }
}
// ORDER 0: PV accumulators rotate (as in the kernel)  1: PV mt-major (two MFMAs in a row on one accumulator)
// ILP: elements of SiLU interleaved (2 in the kernel, 4)
// PHASE 0: MFMA / SiLU interleaved per chunk  1: all MFMAs of a block first, then its SiLU share
// READS 1: LDS operand reads; 0: operands from registers, perturbed per iteration so that nothing is loop-invariant
template <int WPB, int BPC, int RW, int READS, bool BAR, int ORDER, int ILP, int PHASE, int SILU, int LOOKT = 2>
__global__ __launch_bounds__(WPB * 64) __attribute__((amdgpu_waves_per_eu((WPB * BPC) / 4, (WPB * BPC) / 4)))
void k(float* out, unsigned long long* clk, int iters, float c_exp) {
  constexpr int THREADS = WPB * 64;
  __shared__ __attribute__((aligned(16))) uint16_t lk[4096 * 4];
  __shared__ __attribute__((aligned(16))) uint16_t lv[4096 * 4];
  __shared__ uint16_t pad[BPC == 1 ? 30000 : 4000];
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
  auto silu_n = [&](const f32x16& s, int first, uint32_t* pk) {  // ILP elements starting at element `first` (pairs first/2 ..)
    if (SILU == 0) { pk[first / 2] ^= 1; return; }
    float t[ILP];
#pragma unroll
    for (int e = 0; e < ILP; ++e) t[e] = s[first + e] * c_exp;
#pragma unroll
    for (int e = 0; e < ILP; ++e) t[e] = __builtin_amdgcn_exp2f(t[e]);
#pragma unroll
    for (int e = 0; e < ILP; ++e) t[e] = 1.0f + t[e];
#pragma unroll
    for (int e = 0; e < ILP; ++e) t[e] = __builtin_amdgcn_rcpf(t[e]);
#pragma unroll
    for (int e = 0; e < ILP; ++e) t[e] = s[first + e] * t[e];
#pragma unroll
    for (int e = 0; e < ILP; e += 2) pk[(first + e) / 2] = pk2(t[e], t[e + 1]);
  };
  // one pair in two pieces with state carried in t0/t1 (FINE interleave)
  float h0 = 0, h1 = 0;
  auto pair_a = [&](const f32x16& s, int i) { h0 = s[2 * i] * c_exp; h1 = s[2 * i + 1] * c_exp; h0 = __builtin_amdgcn_exp2f(h0); h1 = __builtin_amdgcn_exp2f(h1); h0 = 1.0f + h0; };
  auto pair_b = [&](const f32x16& s, int i, uint32_t* pk) { h1 = 1.0f + h1; h0 = __builtin_amdgcn_rcpf(h0); h1 = __builtin_amdgcn_rcpf(h1); pk[i] = pk2(s[2 * i] * h0, s[2 * i + 1] * h1); };
  u32x4 kreg[8], vreg[8];
  for (int c = 0; c < 8; ++c) { kreg[c] = u32x4{1, 2, 3, (uint32_t)c}; vreg[c] = u32x4{5, 6, 7, (uint32_t)c}; }
  auto rk = [&](int it, int c) -> u32x4 {
    if (READS) return *reinterpret_cast<const u32x4*>(&lk[(koff ^ (c * 16)) + (it & 3) * 4096]);
    return kreg[c];
  };
  auto rv = [&](int it, int c) -> u32x4 {
    if (READS) { const uint16_t* p = &lv[voff + (c & 3) * 32 + (c >> 2) * 2048 + (it & 3) * 4096]; u32x2 lo = tr(p), hi = tr(p + 1024); return u32x4{lo[0], lo[1], hi[0], hi[1]}; }
    return vreg[c];
  };
  // chunk c of the PV block -> (k half j2, output tile mt)
  auto pv_j2 = [&](int c) { return ORDER == 0 ? c / 4 : c & 1; };
  auto pv_mt = [&](int c) { return ORDER == 0 ? c & 3 : c >> 1; };
  auto pv_op = [&](int c) { return pv_mt(c) + 4 * pv_j2(c); };  // operand index in the tile
  constexpr int LOOK = LOOKT;
  // SiLU work of chunk c in a block of 8 chunks covering elements [base, base + 8 * RW)
  auto silu_share = [&](f32x16* s_cur, uint32_t (*pk_cur)[8], int half, int c) {
    // per block: RW * 8 elements = RW * 8 / ILP groups over 8 chunks
    constexpr int GROUPS = RW * 8 / ILP;  // groups per block
    if (GROUPS >= 8) {
#pragma unroll
      for (int g = c * GROUPS / 8; g < (c + 1) * GROUPS / 8; ++g) { int el = g * ILP; silu_n(s_cur[el / 8], half * 8 + el % 8, pk_cur[el / 8]); }
    } else {
      constexpr int EVERY = 8 / GROUPS;
      if (c % EVERY == 0) { int g = c / EVERY; int el = g * ILP; silu_n(s_cur[el / 8], half * 8 + el % 8, pk_cur[el / 8]); }
    }
  };
  unsigned long long t0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
    if (!READS) { kreg[0][0] += 1; vreg[0][0] += 1; }
#pragma unroll
    for (int par = 0; par < 2; ++par) {
      f32x16* s_cur = par ? s_b : s_a; f32x16* s_nxt = par ? s_a : s_b;
      uint32_t (*pk_cur)[8] = par ? pb : pa; uint32_t (*pk_prev)[8] = par ? pa : pb;
      u32x4 vop[8];
#pragma unroll
      for (int c = 0; c < LOOK; ++c) vop[c] = rv(it, pv_op(c));
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int c = 0; c < 8; ++c) {
#pragma unroll
        for (int r = 0; r < RW; ++r) {
          const int j2 = pv_j2(c);
          u32x4 p4 = {pk_prev[r][4 * j2], pk_prev[r][4 * j2 + 1], pk_prev[r][4 * j2 + 2], pk_prev[r][4 * j2 + 3]};
          o[r][pv_mt(c)] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vop[c]), __builtin_bit_cast(bf16x8, p4), o[r][pv_mt(c)], 0, 0, 0);
          if (PHASE == 2) {
            if (r == 0) { if (c + LOOK < 8) vop[c + LOOK] = rv(it, pv_op(c + LOOK)); pair_a(s_cur[c & 1], c / 2); }
            else pair_b(s_cur[c & 1], c / 2, pk_cur[c & 1]);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        if (PHASE != 2 && c + LOOK < 8) vop[c + LOOK] = rv(it, pv_op(c + LOOK));
        if (PHASE == 0) { silu_share(s_cur, pk_cur, 0, c); __builtin_amdgcn_sched_barrier(0); }
      }
      if (PHASE == 1) {
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < 8; ++c) silu_share(s_cur, pk_cur, 0, c);
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
          if (PHASE == 2) {
            if (r == 0) { if (c + LOOK < 8) kop[c + LOOK] = rk(it, c + LOOK); pair_a(s_cur[c & 1], 4 + c / 2); }
            else pair_b(s_cur[c & 1], 4 + c / 2, pk_cur[c & 1]);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        if (PHASE != 2 && c + LOOK < 8) kop[c + LOOK] = rk(it, c + LOOK);
        if (PHASE == 0) { silu_share(s_cur, pk_cur, 1, c); __builtin_amdgcn_sched_barrier(0); }
      }
      if (PHASE == 1) {
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < 8; ++c) silu_share(s_cur, pk_cur, 1, c);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (BAR) { __builtin_amdgcn_sched_barrier(0); __builtin_amdgcn_s_barrier(); __builtin_amdgcn_sched_barrier(0); }
    }
  }
  unsigned long long t1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
  if (tid == 0) { clk[blockIdx.x * 2] = t1 - t0; clk[blockIdx.x * 2 + 1] = r1 - r0; }
  float r = 0; for (int w = 0; w < RW; ++w) { for (int m = 0; m < 4; ++m) for (int i = 0; i < 16; ++i) r += o[w][m][i]; for (int i = 0; i < 8; ++i) r += pa[w][i] + pb[w][i]; r += s_a[w][0] + s_b[w][1]; }
  out[blockIdx.x * THREADS + tid] = r + pad[5];
}
template <int WPB, int BPC, int RW, int READS, bool BAR, int ORDER, int ILP, int PHASE, int SILU, int LOOKT = 2> int run(const char* note) {
  float* out; CK(hipMalloc(&out, 2048 * 512 * 4));
  unsigned long long* clk; CK(hipMalloc(&clk, 1024 * 16)); CK(hipMemset(clk, 0, 1024 * 16));
  int iters = 3000; int blocks = 256 * BPC;
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  k<WPB, BPC, RW, READS, BAR, ORDER, ILP, PHASE, SILU, LOOKT><<<blocks, WPB * 64>>>(out, clk, 30, -0.1f); CK(hipDeviceSynchronize());
  CK(hipEventRecord(e0)); k<WPB, BPC, RW, READS, BAR, ORDER, ILP, PHASE, SILU, LOOKT><<<blocks, WPB * 64>>>(out, clk, iters, -0.1f); CK(hipEventRecord(e1)); CK(hipDeviceSynchronize());
  float ms; CK(hipEventElapsedTime(&ms, e0, e1));
  static unsigned long long h[1024]; CK(hipMemcpy(h, clk, blocks * 16, hipMemcpyDeviceToHost));
  double cmin = 1e30, cmax = 0, rmin = 1e30, rmax = 0;
  for (int b = 0; b < blocks; ++b) { double c = h[2 * b], r = h[2 * b + 1]; cmin = c < cmin ? c : cmin; cmax = c > cmax ? c : cmax; rmin = r < rmin ? r : rmin; rmax = r > rmax ? r : rmax; }
  double subtiles_per_simd = (double)BPC * WPB * RW / 4.0;
  double per = (iters * 2) * subtiles_per_simd;
  printf("look=%d wpb=%d bpc=%d rw=%d reads=%d bar=%d order=%d ilp=%d phase=%d silu=%d : %4.0f ns (blocks: %4.0f..%4.0f ns by realtime), %4.0f..%4.0f clk per sub-tile per SIMD -> %.2f..%.2f GHz  %s\n",
         LOOKT, WPB, BPC, RW, READS, (int)BAR, ORDER, ILP, PHASE, SILU, ms * 1e6 / per, rmin * 10.0 / per, rmax * 10.0 / per, cmin / per, cmax / per, cmin / (rmin * 10.0), cmax / (rmax * 10.0), note);
  fflush(stdout);
  CK(hipFree(out)); CK(hipFree(clk)); return 0;
}
int main() {
  run<4, 2, 1, 1, true, 0, 2, 0, 1>("the persistent kernel's shape");
  run<4, 1, 2, 1, true, 0, 2, 0, 1>("64 rows, one wave per SIMD, MFMA MFMA pair");
  run<4, 1, 2, 1, true, 0, 2, 2, 1>("64 rows, one wave per SIMD, MFMA half-pair MFMA half-pair");
  run<4, 1, 2, 1, false, 0, 2, 2, 1>("  same, no barrier");
  run<4, 1, 2, 1, true, 1, 2, 2, 1>("  same, PV mt-major");
  run<4, 1, 2, 1, true, 0, 2, 2, 1, 3>("  same, lookahead 3");
  run<4, 1, 2, 1, true, 0, 2, 2, 1, 4>("  same, lookahead 4");
  run<4, 1, 2, 0, false, 0, 2, 2, 1>("  same, operands from registers, no barrier");
  run<4, 1, 2, 1, true, 0, 2, 2, 0>("  same, no SiLU");
  run<2, 2, 2, 1, true, 0, 2, 2, 1>("64 rows, two 2-wave blocks per CU, fine interleave");
  return 0;
}
