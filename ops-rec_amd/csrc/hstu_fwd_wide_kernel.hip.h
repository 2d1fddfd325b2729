// HSTU jagged attention forward for gfx950: bf16 / fp16 inputs with head dims in (256, 512].
//
// The reference takes head dims up to 512 (ascendc/attention/hstu_v1/hstu_forward_v1/op_host/tiling_policy.cpp:68-93,
// blockK up to 512 in op_host/atlas950/tiling_policy_arch.cpp:173-177).  The tuned kernel stops at 256: 128 output
// registers per 32 rows, and two four-slot LDS rings of 16 KB sub-tiles.  This kernel carries the same arithmetic to
// 512 on the matrix pipe with a plain structure -- one workgroup per 128-row query tile and window of 256 output dims
// (blockIdx.y: a head dim of v above 256 takes two workgroups per tile, each computing the scores for itself), 32-key
// sub-tiles of K and V in two LDS stages, the next sub-tile on its way while the products of this one run -- and the
// tuned kernel's operand layouts: S^T = K . Q^T with v_mfma_f32_32x32x16 (the Q rows of a lane in 128 registers, K rows read from
// LDS 16 bytes at a time), P^T packed in registers as the B operand of O^T += V^T . P^T, V^T taken from the row-major
// V sub-tile by transposed LDS reads.  LDS rows are padded instead of swizzled (K rows by 16 bytes: the 16 rows an
// operand read takes together fall into different bank groups; V rows by 64 bytes: the four rows of a transposed read
// likewise), so that every LDS address is one per-lane base plus a compile-time offset -- with 384 registers already
// spoken for there is no room for a table of swizzled addresses.  A wavefront holds 128 output, 128 Q and 32 score registers: one wavefront
// per SIMD.  (With all 512 output dims in one wavefront -- 256 output registers -- the compiler kept 156 registers of Q
// rows in scratch memory and a sub-tile's loads were waited for in the open: 89 .. 121 TFLOP/s.)  Head dims are padded to 512 (chunks past the real dims read
// as zeros); a q/k head dim that is not a multiple of 8 stays with the generic kernel.
#pragma once
#include "hstu_fwd_kernel.hip.h"

namespace hstu {

constexpr int kWideDim = 512;

template <typename Tag, bool HAS_RAB, bool HAS_MASK>
__global__ __launch_bounds__(256, 1) void hstu_fwd_wide_kernel(const FwdArgs a)
{
    constexpr int kThreads = 256;
    constexpr int D = kWideDim;
    constexpr int BN = 32;              // keys per LDS tile = one 32-key sub-tile
    constexpr int K_ROW = D + 8;        // elements per K row in LDS (1040 bytes)
    constexpr int V_ROW = D + 32;       // elements per V row in LDS (1088 bytes)
    constexpr int LPW = BN / 4;         // a load instruction fills one row (1 KiB): rows per wavefront and tile
    constexpr int KSTEPS = D / 16;
    constexpr int MTILES = D / 32;

    constexpr int OW = 256;             // output dims per workgroup
    constexpr int MT_O = OW / 32;
    // two stages (separate arrays, so that the compiler can tell the one being filled from the one being read); a V row
    // keeps the pitch of 512 dims, of which the window's 256 are filled
    __shared__ __attribute__((aligned(16))) uint16_t s_k0[BN * K_ROW];
    __shared__ __attribute__((aligned(16))) uint16_t s_k1[BN * K_ROW];
    __shared__ __attribute__((aligned(16))) uint16_t s_v0[BN * V_ROW];
    __shared__ __attribute__((aligned(16))) uint16_t s_v1[BN * V_ROW];

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
    const int ow0 = static_cast<int>(blockIdx.y) * OW;  // first output dim of this workgroup

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

    uint16_t* const out16 = static_cast<uint16_t*>(a.out);
    if (qt == 0 && ow0 == 0) {  // rows past the last offset belong to no sequence: zero-fill them
        const int64_t last = load_index(a.offs_q, a.n_batch, a.idx64);
        const int64_t first_tail = last < 0 ? 0 : last;
        const int64_t row_elems = static_cast<int64_t>(a.n_heads_q) * a.d_v;
        const int64_t n_tail = (a.total_q > first_tail ? a.total_q - first_tail : 0) * row_elems;
        uint16_t* tail = out16 + first_tail * row_elems;
        for (int64_t e = static_cast<int64_t>(bhid) * kThreads + tid; e < n_tail;
             e += static_cast<int64_t>(a.bh) * kThreads) {
            tail[e] = 0;
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
    // (.../op_kernel/atlas950/hstu_dense_causal_mask.h:186-260)
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

    const uint32_t q_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_qk * 2u;
    const uint32_t k_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_qk * 2u;
    const uint32_t v_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_v * 2u;
    const uint32_t o_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_v * 2u;
    const __amdgpu_buffer_rsrc_t q_rsrc =
        make_rsrc(static_cast<const uint16_t*>(a.q) + (q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_qk),
                  static_cast<uint32_t>(sq - 1) * q_stride + a.d_qk * 2u);
    const __amdgpu_buffer_rsrc_t k_rsrc =
        make_rsrc(static_cast<const uint16_t*>(a.k) + (k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_qk),
                  sk > 0 ? static_cast<uint32_t>(sk - 1) * k_stride + a.d_qk * 2u : 0u);
    const __amdgpu_buffer_rsrc_t v_rsrc =
        make_rsrc(static_cast<const uint16_t*>(a.v) + (k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_v),
                  sk > 0 ? static_cast<uint32_t>(sk - 1) * v_stride + a.d_v * 2u : 0u);
    const __amdgpu_buffer_rsrc_t o_rsrc = make_rsrc(out16 + (q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_v),
                                                    static_cast<uint32_t>(sq - 1) * o_stride + a.d_v * 2u);

    // Q fragment: lane (ln, lh) holds Q[row][16 js + 8 lh .. + 7] for js = 0 .. KSTEPS - 1
    u32x4_t qf[KSTEPS];
    {
        const uint32_t row_off = static_cast<uint32_t>(wr0 + ln) * q_stride;
#pragma unroll
        for (int js = 0; js < KSTEPS; ++js) {
            const int d0 = 16 * js + 8 * lh;
            const uint32_t off = (d0 < a.d_qk) ? row_off + d0 * 2u : kOutOfRange;
            qf[js] = __builtin_amdgcn_raw_buffer_load_b128(q_rsrc, static_cast<int>(off), 0, 0);
        }
    }

    // load instruction i of this wavefront fills row wave * LPW + i of a tile: lane l brings the 16-byte chunk l
    const uint32_t k_lane_src = (lane * 8 < a.d_qk) ? static_cast<uint32_t>(lane) * 16u : kOutOfRange;
    const uint32_t v_lane_src =
        (lane < OW / 8 && ow0 + lane * 8 < a.d_v) ? static_cast<uint32_t>(ow0 + lane * 8) * 2u : kOutOfRange;
    // per-lane bases of the operand reads: K row ln, chunk lh (+ 2 js chunks per MFMA step); V rows vr0 (+ 8, + 16 j2),
    // dims 16 ((lane / 16) % 2) + 4 (lane % 4) (+ 32 mt)
    const int k_read_off = ln * K_ROW + 8 * lh;
    const int v_read_off = (4 * lh + ((lane & 15) >> 2)) * V_ROW + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

    const uint32_t bias_bytes = static_cast<uint32_t>(a.max_q) * static_cast<uint32_t>(a.max_k) * 2u;
    const int64_t bias_plane = (static_cast<int64_t>(b) * a.n_heads_q + h) * a.max_q * static_cast<int64_t>(a.max_k);
    const __amdgpu_buffer_rsrc_t rab_rsrc =
        make_rsrc(HAS_RAB ? static_cast<const uint16_t*>(a.rab) + bias_plane : nullptr, HAS_RAB ? bias_bytes : 0u);
    const __amdgpu_buffer_rsrc_t mask_rsrc =
        make_rsrc(HAS_MASK ? static_cast<const uint16_t*>(a.mask) + bias_plane : nullptr, HAS_MASK ? bias_bytes : 0u);
    const uint32_t bias_row_off = static_cast<uint32_t>(wr0 + ln) * static_cast<uint32_t>(a.max_k) * 2u;
    const bool bias_vec = a.bias_vec_ok != 0;
    // the 16 rab / mask values of this lane's score elements: keys c0 + 8 g + 4 lh + 0..3 of its row
    auto load_bias = [&](__amdgpu_buffer_rsrc_t rsrc, int c0, f32x16_t& w) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const uint32_t off = bias_row_off + static_cast<uint32_t>(c0 + 8 * g + 4 * lh) * 2u;
            if (bias_vec) {
                const u32x2_t t = __builtin_amdgcn_raw_buffer_load_b64(rsrc, static_cast<int>(off), 0, 0);
                w[4 * g + 0] = lo_to_float<Tag>(t[0]);
                w[4 * g + 1] = hi_to_float<Tag>(t[0]);
                w[4 * g + 2] = lo_to_float<Tag>(t[1]);
                w[4 * g + 3] = hi_to_float<Tag>(t[1]);
            } else {
                // (the offset goes through an empty asm so that the optimiser does not relate these element loads
                // to the vector load of the other branch)
                uint32_t eoff = off;
                asm volatile("" : "+v"(eoff));
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t raw = __builtin_amdgcn_raw_buffer_load_b16(rsrc, static_cast<int>(eoff + 2u * e), 0, 0);
                    w[4 * g + e] = lo_to_float<Tag>(raw & 0xffffu);
                }
            }
        }
    };

    f32x16_t o_acc[MT_O];
#pragma unroll
    for (int mt = 0; mt < MT_O; ++mt) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            o_acc[mt][i] = 0.f;
        }
    }
    const float c_exp = a.c_exp;

    // sub-tile kt into a stage (requests past the last sub-tile move nothing)
    auto request = [&](uint16_t* sk_to, uint16_t* sv_to, int kt) {
        const bool past = kt >= n_kt;
        const uint32_t kb = static_cast<uint32_t>(kt * BN) * k_stride;
        const uint32_t vb = static_cast<uint32_t>(kt * BN) * v_stride;
#pragma unroll
        for (int i = 0; i < LPW; ++i) {
            const int r = wave * LPW + i;
            load_to_lds_b128(k_rsrc, sk_to + r * K_ROW, past ? kOutOfRange : k_lane_src + kb + static_cast<uint32_t>(r) * k_stride);
            load_to_lds_b128(v_rsrc, sv_to + r * V_ROW, past ? kOutOfRange : v_lane_src + vb + static_cast<uint32_t>(r) * v_stride);
        }
    };
    // one step: sub-tile kt has landed in (sk, sv) -- mine, then everybody's -- and everybody is done with the other stage,
    // which the next sub-tile may now fill while the products of this one run
    auto step = [&](const uint16_t* sk, const uint16_t* sv, uint16_t* sk_next, uint16_t* sv_next, int kt) {
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        request(sk_next, sv_next, kt + 1);
        const uint16_t* const k_read = sk + k_read_off;
        const uint16_t* const v_read = sv + v_read_off;
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
            // S^T = K . Q^T (one accumulation chain: a second one would cost 16 of the registers the Q rows need)
#pragma unroll
            for (int js = 0; js < KSTEPS; ++js) {
                const u32x4_t ka = *reinterpret_cast<const u32x4_t*>(k_read + 16 * js);
                s = mfma32<Tag>(ka, qf[js], s);
                if (js % 4 == 3) {
                    __builtin_amdgcn_sched_barrier(0);  // (operand reads stay next to their MFMAs)
                }
            }
            // P^T = S^T * sigmoid(alpha * S^T), masked
            const bool full = !HAS_MASK && (c0 + 32 <= wb.lim_min) &&
                              !(wb.any_hole && c0 + 32 > hist_k && c0 < wb.hole_hi_max);
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float sv_ = s[i];
                const float ex = __builtin_amdgcn_exp2f(sv_ * c_exp);
                s[i] = sv_ * __builtin_amdgcn_rcpf(1.0f + ex);
            }
            if (!full) {
                f32x16_t mw;
                if constexpr (HAS_MASK) {
                    load_bias(mask_rsrc, c0, mw);
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int jj = c0 + 8 * (i / 4) + 4 * lh + (i % 4);
                    const bool vis = (jj < lim) && !(jj >= hole_lo && jj < hole_hi);
                    float pv = s[i];
                    if constexpr (HAS_MASK) {
                        pv *= mw[i];
                    }
                    s[i] = vis ? pv : 0.f;
                }
            }
            uint32_t pk[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                pk[i] = pack2<Tag>(s[2 * i], s[2 * i + 1]);
            }
            // O^T += V^T . P^T: chunk (mt, j2) contracts the 16 keys of half j2 into output tile mt of the window
#pragma unroll
            for (int mt = 0; mt < MT_O; ++mt) {
#pragma unroll
                for (int j2 = 0; j2 < 2; ++j2) {
                    const u32x2_t lo = lds_read_tr16_b64(v_read + 32 * mt + 16 * j2 * V_ROW);
                    const u32x2_t hi = lds_read_tr16_b64(v_read + 32 * mt + 16 * j2 * V_ROW + 8 * V_ROW);
                    const u32x4_t va = {lo[0], lo[1], hi[0], hi[1]};
                    const u32x4_t pb = {pk[4 * j2 + 0], pk[4 * j2 + 1], pk[4 * j2 + 2], pk[4 * j2 + 3]};
                    o_acc[mt] = mfma32<Tag>(va, pb, o_acc[mt]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    if (n_kt > 0) {
        request(s_k0, s_v0, 0);
        for (int kt = 0; kt < n_kt; kt += 2) {
            step(s_k0, s_v0, s_k1, s_v1, kt);
            if (kt + 1 >= n_kt) {
                break;
            }
            step(s_k1, s_v1, s_k0, s_v0, kt + 1);
        }
        // (the request past the last sub-tile names a stage: it has moved nothing, and is waited for before the kernel ends)
        __builtin_amdgcn_s_waitcnt(0);
    }

    // store O: lane holds query row (wr0 + ln), dims ow0 + 32 mt + 8 g + 4 lh + 0..3 (d_v is a multiple of 16)
    {
        const float c_out = a.c_out;
        const uint32_t row_off = static_cast<uint32_t>(wr0 + ln) * o_stride;
#pragma unroll
        for (int mt = 0; mt < MT_O; ++mt) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d0 = ow0 + 32 * mt + 8 * g + 4 * lh;
                const uint32_t off = (d0 < a.d_v) ? row_off + d0 * 2u : kOutOfRange;
                u32x2_t w;
                w[0] = pack2<Tag>(o_acc[mt][4 * g + 0] * c_out, o_acc[mt][4 * g + 1] * c_out);
                w[1] = pack2<Tag>(o_acc[mt][4 * g + 2] * c_out, o_acc[mt][4 * g + 3] * c_out);
                __builtin_amdgcn_raw_buffer_store_b64(w, o_rsrc, static_cast<int>(off), 0, 0);
            }
        }
    }
}

}  // namespace hstu
