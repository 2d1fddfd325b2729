// HSTU jagged attention forward for gfx950: fp32 inputs, fp32 output.
//
// Same algorithm and work split as the 16-bit kernel (one workgroup per 128-row query tile, four
// wavefronts of 32 rows, K/V tiles staged in LDS by buffer loads that write LDS directly, S^T = K.Q^T
// so that P^T feeds the second product from registers), but both products run on the fp32 matrix
// instruction v_mfma_f32_32x32x2_f32 and P is not rounded.  This variant exists for dtype coverage
// (the reference accepts fp32 q/k/v: op_host/atlas950/op_def_arch.h:23); it is not the tuned path.
//
// Operand layouts of v_mfma_f32_32x32x2_f32 (A is 32x2, B is 2x32): lane l supplies A[l % 32][l / 32]
// and B[l / 32][l % 32]; the accumulator layout is that of the 32x32 bf16 instruction.
#pragma once
#include "hstu_fwd_kernel.hip.h"

namespace hstu {

// 16-byte chunks of a row are XOR-swizzled by the row number so that "32 lanes = 32 rows, same
// column" reads (the A operand of S^T = K.Q^T) spread over the banks.
template <int D>
__device__ __forceinline__ int f32_chunk_swizzle(int row, int chunk)
{
    constexpr int CPR = D / 4;  // 16-byte chunks per row
    return chunk ^ (row & (CPR - 1) & 31);
}

template <int D, bool HAS_RAB, bool HAS_MASK>
__global__ __launch_bounds__(256, 1) void hstu_fwd_f32_kernel(const FwdArgs a)
{
    constexpr int kThreads = 256;
    constexpr int BN = 32;                       // keys per LDS tile = one 32-key sub-tile
    constexpr int CPR = D / 4;                   // 16-byte chunks per row
    constexpr int TILE_FLOATS = BN * D;
    constexpr int LOADS = TILE_FLOATS / 256 / 4;  // 1 KiB load instructions per wavefront per tile
    static_assert(TILE_FLOATS % 1024 == 0, "tile must split evenly over four wavefronts");
    constexpr int QCHUNKS = D / 8;               // float4 chunks of Q held per lane
    constexpr int MTILES = D / 32;

    __shared__ __attribute__((aligned(1024))) float s_k[TILE_FLOATS];
    __shared__ __attribute__((aligned(1024))) float s_v[TILE_FLOATS];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = uniform(tid >> 6);
    const int ln = lane & 31;
    const int lh = lane >> 5;

    const int lvl = blockIdx.x / a.bh;
    const int bhid = blockIdx.x - lvl * a.bh;
    const int qt = a.n_qtiles - 1 - lvl;
    const int b = bhid / a.n_heads_q;
    const int h = bhid - b * a.n_heads_q;
    const int hk = h / a.head_ratio;

    int64_t q0 = load_index(a.offs_q, b, a.idx64);
    int64_t q1 = load_index(a.offs_q, b + 1, a.idx64);
    int64_t k0 = load_index(a.offs_k, b, a.idx64);
    int64_t k1 = load_index(a.offs_k, b + 1, a.idx64);
    q1 = q1 < a.total_q ? q1 : a.total_q;
    k1 = k1 < a.total_k ? k1 : a.total_k;
    q0 = q0 < 0 ? 0 : q0;
    k0 = k0 < 0 ? 0 : k0;
    int sq = static_cast<int>(q1 > q0 ? q1 - q0 : 0);
    int sk = static_cast<int>(k1 > k0 ? k1 - k0 : 0);
    sq = uniform(sq < a.max_q ? sq : a.max_q);
    sk = uniform(sk < a.max_k ? sk : a.max_k);

    float* const out32 = static_cast<float*>(a.out);
    if (qt == 0) {  // rows past the last offset belong to no sequence: zero-fill them
        const int64_t last = load_index(a.offs_q, a.n_batch, a.idx64);
        const int64_t first_tail = last < 0 ? 0 : last;
        const int64_t row_elems = static_cast<int64_t>(a.n_heads_q) * a.d_v;
        const int64_t n_tail = (a.total_q > first_tail ? a.total_q - first_tail : 0) * row_elems;
        float* tail = out32 + first_tail * row_elems;
        for (int64_t e = static_cast<int64_t>(bhid) * kThreads + tid; e < n_tail;
             e += static_cast<int64_t>(a.bh) * kThreads) {
            tail[e] = 0.f;
        }
    }

    const int r0 = qt * kBlockM;
    if (r0 >= sq) {
        return;
    }
    const int wr0 = r0 + wave * kWaveM;
    const bool wave_active = wr0 < sq;

    int n_ctx = 0;
    int n_tgt = 0;
    if (a.mask_type == 0) {
        if (a.num_ctx) {
            n_ctx = static_cast<int>(load_index(a.num_ctx, b, a.idx64));
        }
        if (a.num_tgt) {
            n_tgt = static_cast<int>(load_index(a.num_tgt, b, a.idx64));
        }
        n_ctx = uniform(n_ctx < 0 ? 0 : n_ctx);
        n_tgt = uniform(n_tgt < 0 ? 0 : (n_tgt > sk ? sk : n_tgt));
    }
    const int delta = sk - sq;
    const int hist_k = sk - n_tgt;

    // per-row visibility: visible(j) = j < lim && !(hole_lo <= j < hole_hi)
    int row = wr0 + ln;
    row = row < sq - 1 ? row : sq - 1;
    int lim;
    int hole_lo = 0;
    int hole_hi = 0;
    if (a.mask_type == 0) {
        lim = row + delta + 1;
        if (row < n_ctx) {
            lim = lim > hist_k ? lim : hist_k;
        }
        lim = lim < 0 ? 0 : (lim > sk ? sk : lim);
        if (n_tgt > 0 && a.target_group > 0) {
            const int ti = row - (sq - n_tgt);
            if (ti >= 0) {
                hole_lo = hist_k;
                hole_hi = hist_k + (ti / a.target_group) * a.target_group;
            }
        }
    } else {
        lim = sk;
    }
    const WaveBounds wb = wave_bounds(a.mask_type, wr0, sq, sk, n_ctx, n_tgt, a.target_group, wave_active);

    int kmax;
    if (a.mask_type == 0) {
        const int r1 = (r0 + kBlockM < sq) ? r0 + kBlockM : sq;
        kmax = r1 + delta;
        if (r0 < n_ctx) {
            kmax = kmax > hist_k ? kmax : hist_k;
        }
        kmax = kmax < 0 ? 0 : (kmax > sk ? sk : kmax);
    } else {
        kmax = sk;
    }
    const int n_kt = uniform((kmax + BN - 1) / BN);

    const uint32_t q_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_qk * 4u;
    const uint32_t k_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_qk * 4u;
    const uint32_t v_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_v * 4u;
    const uint32_t o_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_v * 4u;
    const __amdgpu_buffer_rsrc_t q_rsrc =
        make_rsrc(static_cast<const float*>(a.q) + (q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_qk),
                  static_cast<uint32_t>(sq - 1) * q_stride + a.d_qk * 4u);
    const __amdgpu_buffer_rsrc_t k_rsrc =
        make_rsrc(static_cast<const float*>(a.k) + (k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_qk),
                  sk > 0 ? static_cast<uint32_t>(sk - 1) * k_stride + a.d_qk * 4u : 0u);
    const __amdgpu_buffer_rsrc_t v_rsrc =
        make_rsrc(static_cast<const float*>(a.v) + (k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_v),
                  sk > 0 ? static_cast<uint32_t>(sk - 1) * v_stride + a.d_v * 4u : 0u);
    const __amdgpu_buffer_rsrc_t o_rsrc = make_rsrc(out32 + (q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_v),
                                                    static_cast<uint32_t>(sq - 1) * o_stride + a.d_v * 4u);

    // Q fragment: MFMA step 4*j + e of the QK product contracts head-dim element 4*(2j + lh) + e, so a
    // lane holds the float4 chunks 2j + lh of its row (the contraction order is free, K follows it)
    typedef __attribute__((ext_vector_type(4))) float f32x4_t;
    f32x4_t qf[QCHUNKS];
    {
        const uint32_t row_off = static_cast<uint32_t>(wr0 + ln) * q_stride;
#pragma unroll
        for (int j = 0; j < QCHUNKS; ++j) {
            const int d0 = 4 * (2 * j + lh);
            const uint32_t off = (d0 < a.d_qk) ? row_off + d0 * 4u : kOutOfRange;
            qf[j] = __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(q_rsrc, static_cast<int>(off), 0, 0));
        }
    }

    uint32_t k_src[LOADS];
    uint32_t v_src[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        const int slot = (wave * LOADS + i) * 64 + lane;
        const int r = slot / CPR;
        const int pc = slot - r * CPR;
        const int c = f32_chunk_swizzle<D>(r, pc);
        k_src[i] = (c * 4 < a.d_qk) ? static_cast<uint32_t>(r) * k_stride + c * 16u : kOutOfRange;
        v_src[i] = (c * 4 < a.d_v) ? static_cast<uint32_t>(r) * v_stride + c * 16u : kOutOfRange;
    }

    const uint32_t bias_bytes = static_cast<uint32_t>(a.max_q) * static_cast<uint32_t>(a.max_k) * 4u;
    const int64_t bias_plane = (static_cast<int64_t>(b) * a.n_heads_q + h) * a.max_q * static_cast<int64_t>(a.max_k);
    const __amdgpu_buffer_rsrc_t rab_rsrc =
        make_rsrc(HAS_RAB ? static_cast<const float*>(a.rab) + bias_plane : nullptr, HAS_RAB ? bias_bytes : 0u);
    const __amdgpu_buffer_rsrc_t mask_rsrc =
        make_rsrc(HAS_MASK ? static_cast<const float*>(a.mask) + bias_plane : nullptr, HAS_MASK ? bias_bytes : 0u);
    const uint32_t bias_row_off = static_cast<uint32_t>(wr0 + ln) * static_cast<uint32_t>(a.max_k) * 4u;
    const bool bias_vec = a.bias_vec_ok != 0;
    auto load_bias = [&](__amdgpu_buffer_rsrc_t rsrc, int c0, f32x16_t& w) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const uint32_t off = bias_row_off + static_cast<uint32_t>(c0 + 8 * g + 4 * lh) * 4u;
            if (bias_vec) {
                // (the result is reinterpreted as a float vector before its elements are taken: taking
                // integer elements straight from this builtin's result is narrowed to a one-element load
                // by the optimiser of this toolchain)
                const f32x4_t t = __builtin_bit_cast(
                    f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, static_cast<int>(off), 0, 0));
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    w[4 * g + e] = t[e];
                }
            } else {
                // the offset is laundered through an empty asm so that the optimiser cannot relate these
                // element loads to the vector load of the other branch (it otherwise folds the two and
                // replicates the first element)
                uint32_t eoff = off;
                asm volatile("" : "+v"(eoff));
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    w[4 * g + e] = __builtin_bit_cast(
                        float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, static_cast<int>(eoff + 4u * e), 0, 0));
                }
            }
        }
    };

    f32x16_t o_acc[MTILES];
#pragma unroll
    for (int mt = 0; mt < MTILES; ++mt) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            o_acc[mt][i] = 0.f;
        }
    }
    const float c_exp = a.c_exp;

    for (int kt = 0; kt < n_kt; ++kt) {
        const uint32_t kb = static_cast<uint32_t>(kt * BN) * k_stride;
        const uint32_t vb = static_cast<uint32_t>(kt * BN) * v_stride;
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(k_rsrc, (__attribute__((address_space(3))) void*)(s_k + (wave * LOADS + i) * 256),
                                                     16, static_cast<int>(k_src[i] + kb), 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(v_rsrc, (__attribute__((address_space(3))) void*)(s_v + (wave * LOADS + i) * 256),
                                                     16, static_cast<int>(v_src[i] + vb), 0, 0, 0);
        }
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();

        const int c0 = kt * BN;
        if (c0 < wb.lim_max) {
            f32x16_t s;
            if constexpr (HAS_RAB) {
                load_bias(rab_rsrc, c0, s);
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    s[i] = 0.f;
                }
            }
            f32x16_t mw;
            if constexpr (HAS_MASK) {
                load_bias(mask_rsrc, c0, mw);
            }
            // S^T = K . Q^T
#pragma unroll
            for (int j = 0; j < QCHUNKS; ++j) {
                const f32x4_t kc =
                    *reinterpret_cast<const f32x4_t*>(s_k + ln * D + f32_chunk_swizzle<D>(ln, 2 * j + lh) * 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    s = __builtin_amdgcn_mfma_f32_32x32x2f32(kc[e], qf[j][e], s, 0, 0, 0);
                }
            }
            // P^T = S^T * sigmoid(alpha * S^T), masked
            const bool full = !HAS_MASK && (c0 + 32 <= wb.lim_min) &&
                              !(wb.any_hole && c0 + 32 > hist_k && c0 < wb.hole_hi_max);
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float sv = s[i];
                const float ex = __builtin_amdgcn_exp2f(sv * c_exp);
                s[i] = sv * __builtin_amdgcn_rcpf(1.0f + ex);
            }
            if (!full) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int jj = c0 + 8 * (i / 4) + 4 * lh + (i % 4);
                    const bool vis = (jj < lim) && !(jj >= hole_lo && jj < hole_hi);
                    float p = s[i];
                    if constexpr (HAS_MASK) {
                        p *= mw[i];
                    }
                    s[i] = vis ? p : 0.f;
                }
            }
            // O^T += V^T . P^T : step i contracts the key pair {8 (i/4) + i % 4, same + 4}, one per lane half
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int vr = 8 * (i / 4) + 4 * lh + (i % 4);
#pragma unroll
                for (int mt = 0; mt < MTILES; ++mt) {
                    const int col = 32 * mt + ln;
                    const float va = s_v[vr * D + f32_chunk_swizzle<D>(vr, col >> 2) * 4 + (col & 3)];
                    o_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(va, s[i], o_acc[mt], 0, 0, 0);
                }
            }
        }
        __syncthreads();
    }

    // store O: lane holds query row (wr0 + ln), dims 32 mt + 8 g + 4 lh + 0..3
    {
        const float c_out = a.c_out;
        const uint32_t row_off = static_cast<uint32_t>(wr0 + ln) * o_stride;
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d0 = 32 * mt + 8 * g + 4 * lh;
                const uint32_t off = (d0 < a.d_v) ? row_off + d0 * 4u : kOutOfRange;
                u32x4_t w;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    w[e] = __builtin_bit_cast(uint32_t, o_acc[mt][4 * g + e] * c_out);
                }
                __builtin_amdgcn_raw_buffer_store_b128(w, o_rsrc, static_cast<int>(off), 0, 0);
            }
        }
    }
}

}  // namespace hstu
