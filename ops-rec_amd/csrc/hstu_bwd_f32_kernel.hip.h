// HSTU jagged attention backward for gfx950: fp32 inputs, fp32 gradients, head dims up to 128.
//
//   X = alpha (Q K^T + rab),  sig = sigmoid(X),  P = X sig scale M,
//   dV = P^T dO,  dP = dO V^T,  dS = alpha scale M dP sig (1 + X (1 - sig)),  d rab = dS,  dQ = dS K,  dK = dS^T Q
// (ascendc/attention/hstu_v1/hstu_backward_v1/op_kernel/vector_score.h:159-205; the reference's backward takes fp32,
// hstu_backward_v1/op_host).  The backward's counterpart of hstu_fwd_f32_kernel: every product on the fp32 matrix
// instruction v_mfma_f32_32x32x2_f32, nothing rounded on the way, the plain structure of that kernel (one 32-row
// sub-tile of the streamed operands in LDS at a time: load / barrier / products / barrier), and the split of the
// 16-bit backward into two kernels without atomics:
//
//   hstu_bwd_f32_dq_kernel   one workgroup per 128-row query tile of one (sequence, head); a wavefront keeps its 32
//                            Q and dO rows in registers, K and V sub-tiles pass through LDS:
//                              S^T = K . Q^T,  dP^T = V . dO^T  (lane = query row, registers = keys),
//                              dS^T in registers, stored as d rab when asked for,  dQ^T += K^T . dS^T
//   hstu_bwd_f32_dkv_kernel  one workgroup per 128-key tile of one (sequence, K/V head); a wavefront keeps its 32 K
//                            and V rows in registers, the Q and dO sub-tiles of every query head of the group pass
//                            through LDS:
//                              S = Q . K^T,  dP = dO . V^T  (lane = key, registers = query rows),
//                              dV^T += dO^T . P,  dK^T += Q^T . dS
// In both, the score block comes out of the matrix pipe in the layout in which the products that consume it want
// their B operand (one value per lane and MFMA), as in the forward.  The host clears dq, dk, dv and d rab ahead of the
// launches, so the kernels write what they compute and nothing else.
//
// Operand layouts of v_mfma_f32_32x32x2_f32 (A is 32x2, B is 2x32): lane l supplies A[l % 32][l / 32] and
// B[l / 32][l % 32]; accumulator element e of lane l is row 8 (e / 4) + 4 (l / 32) + e % 4, column l % 32.
#pragma once
#include "hstu_bwd_kernel.hip.h"
#include "hstu_fwd_f32_kernel.hip.h"

namespace hstu {

typedef __attribute__((ext_vector_type(4))) float bwd_f32x4_t;

// the 16 values of a [max_q, max_k] fp32 plane at row `row`, keys c0 + 8 g + 4 half + 0..3 (g = 0..3): the elements of
// a lane in the S^T layout (lane = query row)
__device__ __forceinline__ void f32_load_row_keys(__amdgpu_buffer_rsrc_t rsrc, uint32_t row_off, int c0, int half, int max_k,
                                                  bool vec, f32x16_t& w)
{
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const int key = c0 + 8 * g + 4 * half;
        const uint32_t off = row_off + static_cast<uint32_t>(key) * 4u;
        if (vec) {
            const bwd_f32x4_t t = __builtin_bit_cast(
                bwd_f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, static_cast<int>(key < max_k ? off : kOutOfRange), 0, 0));
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                w[4 * g + e] = t[e];
            }
        } else {
            uint32_t eoff = off;
            asm volatile("" : "+v"(eoff));  // (keeps the optimiser from folding these into the vector load above)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                w[4 * g + e] = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, static_cast<int>(key + e < max_k ? eoff + 4u * e : kOutOfRange), 0, 0));
            }
        }
    }
}

// PLANES: dS and P are stored as well, for a key-tile kernel that reads them back instead of computing them again: per
// query row and 32-key block the 32 dS values followed by the 32 P values (a.p_plane; fp32; nothing in it is cleared:
// the reading kernel reads what this one wrote).
template <int D, bool HAS_RAB, bool HAS_MASK, bool PLANES = false>
__global__ __launch_bounds__(256, 1) void hstu_bwd_f32_dq_kernel(const BwdArgs a)
{
    constexpr int BN = 32;
    constexpr int CPR = D / 4;  // 16-byte chunks per row
    constexpr int TILE_FLOATS = BN * D;
    constexpr int LOADS = TILE_FLOATS / 256 / 4;  // 1 KiB load instructions per wavefront per tile
    static_assert(TILE_FLOATS % 1024 == 0, "tile must split evenly over four wavefronts");
    constexpr int QCHUNKS = D / 8;  // float4 chunks of a row held per lane
    constexpr int MTILES = D / 32;

    __shared__ __attribute__((aligned(1024))) float s_k[TILE_FLOATS];
    __shared__ __attribute__((aligned(1024))) float s_v[TILE_FLOATS];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = uniform(tid >> 6);
    const int ln = lane & 31;
    const int lh = lane >> 5;
    const int per_level = a.n_batch * a.n_heads_q;
    const int lvl = blockIdx.x / per_level;
    const int rem = blockIdx.x - lvl * per_level;
    const int qt = a.n_qtiles - 1 - lvl;
    const int b = rem / a.n_heads_q;
    const int h = rem - b * a.n_heads_q;
    const int hk = h / a.head_ratio;
    const SeqInfo si = load_seq(a, b);
    const int sq = uniform(si.sq), sk = uniform(si.sk);
    const int r0 = qt * kBlockM;
    if (r0 >= sq) {
        return;
    }
    const int wr0 = r0 + wave * kWaveM;
    int row = wr0 + ln;
    row = row < sq - 1 ? row : sq - 1;
    int lim, hole_lo, hole_hi;
    row_bounds(si, a.mask_type, a.target_group, row, lim, hole_lo, hole_hi);
    const WaveBounds wb = wave_bounds(a.mask_type, wr0, sq, sk, si.n_ctx, si.n_tgt, a.target_group, wr0 < sq);
    int kmax;
    if (a.mask_type == 0) {
        const int r1 = (r0 + kBlockM < sq) ? r0 + kBlockM : sq;
        kmax = r1 + si.delta;
        if (r0 < si.n_ctx) {
            kmax = kmax > si.hist_k ? kmax : si.hist_k;
        }
        kmax = kmax < 0 ? 0 : (kmax > sk ? sk : kmax);
    } else {
        kmax = sk;
    }
    const int n_kt = uniform((kmax + BN - 1) / BN);

    const uint32_t q_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_qk * 4u;
    const uint32_t g_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_v * 4u;
    const uint32_t k_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_qk * 4u;
    const uint32_t v_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_v * 4u;
    const __amdgpu_buffer_rsrc_t q_rsrc =
        make_rsrc(static_cast<const float*>(a.q) + (si.q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_qk),
                  static_cast<uint32_t>(sq - 1) * q_stride + a.d_qk * 4u);
    const __amdgpu_buffer_rsrc_t g_rsrc =
        make_rsrc(static_cast<const float*>(a.grad) + (si.q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_v),
                  static_cast<uint32_t>(sq - 1) * g_stride + a.d_v * 4u);
    const __amdgpu_buffer_rsrc_t dq_rsrc =
        make_rsrc(static_cast<float*>(a.dq) + (si.q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_qk),
                  static_cast<uint32_t>(sq - 1) * q_stride + a.d_qk * 4u);
    const __amdgpu_buffer_rsrc_t k_rsrc =
        make_rsrc(static_cast<const float*>(a.k) + (si.k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_qk),
                  sk > 0 ? static_cast<uint32_t>(sk - 1) * k_stride + a.d_qk * 4u : 0u);
    const __amdgpu_buffer_rsrc_t v_rsrc =
        make_rsrc(static_cast<const float*>(a.v) + (si.k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_v),
                  sk > 0 ? static_cast<uint32_t>(sk - 1) * v_stride + a.d_v * 4u : 0u);

    // Q and dO fragments: MFMA step 4 j + e contracts head-dim element 4 (2 j + lh) + e (see the forward)
    bwd_f32x4_t qf[QCHUNKS], gf[QCHUNKS];
    {
        const uint32_t q_off = static_cast<uint32_t>(wr0 + ln) * q_stride;
        const uint32_t g_off = static_cast<uint32_t>(wr0 + ln) * g_stride;
#pragma unroll
        for (int j = 0; j < QCHUNKS; ++j) {
            const int d0 = 4 * (2 * j + lh);
            qf[j] = __builtin_bit_cast(bwd_f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(
                                                        q_rsrc, static_cast<int>(d0 < a.d_qk ? q_off + d0 * 4u : kOutOfRange), 0, 0));
            gf[j] = __builtin_bit_cast(bwd_f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(
                                                        g_rsrc, static_cast<int>(d0 < a.d_v ? g_off + d0 * 4u : kOutOfRange), 0, 0));
        }
    }
    uint32_t k_src[LOADS], v_src[LOADS];
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
    const bool want_drab = HAS_RAB && a.drab != nullptr;
    const __amdgpu_buffer_rsrc_t drab_rsrc =
        make_rsrc(want_drab ? static_cast<float*>(a.drab) + bias_plane : nullptr, want_drab ? bias_bytes : 0u);
    const uint32_t pair_pitch = 64u * static_cast<uint32_t>((a.max_k + 31) / 32);  // elements per row of the dS / P plane
    const __amdgpu_buffer_rsrc_t pair_rsrc = make_rsrc(
        PLANES ? static_cast<float*>(a.p_plane) + (static_cast<int64_t>(b) * a.n_heads_q + h) * a.max_q * static_cast<int64_t>(pair_pitch) : nullptr,
        PLANES ? static_cast<uint32_t>(a.max_q) * pair_pitch * 4u : 0u);
    const uint32_t pair_row_off = (wr0 + ln < sq) ? static_cast<uint32_t>(wr0 + ln) * pair_pitch * 4u : kOutOfRange;
    // rows past the sequence lie inside the plane but are not read or written: their offset leaves it
    const uint32_t bias_row_off =
        (wr0 + ln < sq) ? static_cast<uint32_t>(wr0 + ln) * static_cast<uint32_t>(a.max_k) * 4u : kOutOfRange;
    const bool bias_vec = a.bias_vec_ok != 0;

    f32x16_t dq_acc[MTILES];
#pragma unroll
    for (int mt = 0; mt < MTILES; ++mt) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            dq_acc[mt][i] = 0.f;
        }
    }
    const ScoreConsts sconst = score_consts(a.alpha, a.scale);

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
        if (c0 < swept_key_limit(a, si, wr0)) {
            f32x16_t s, dp;
            if constexpr (HAS_RAB) {
                f32_load_row_keys(rab_rsrc, bias_row_off, c0, lh, a.max_k, bias_vec, s);
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    s[i] = 0.f;
                }
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                dp[i] = 0.f;
            }
            f32x16_t mw;
            if constexpr (HAS_MASK) {
                f32_load_row_keys(mask_rsrc, bias_row_off, c0, lh, a.max_k, bias_vec, mw);
            }
            // S^T = K . Q^T and dP^T = V . dO^T
#pragma unroll
            for (int j = 0; j < QCHUNKS; ++j) {
                const int at = ln * D + f32_chunk_swizzle<D>(ln, 2 * j + lh) * 4;
                const bwd_f32x4_t kc = *reinterpret_cast<const bwd_f32x4_t*>(s_k + at);
                const bwd_f32x4_t vc = *reinterpret_cast<const bwd_f32x4_t*>(s_v + at);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    s = __builtin_amdgcn_mfma_f32_32x32x2f32(kc[e], qf[j][e], s, 0, 0, 0);
                    dp = __builtin_amdgcn_mfma_f32_32x32x2f32(vc[e], gf[j][e], dp, 0, 0, 0);
                }
            }
            // dS^T, masked
            const bool full = !HAS_MASK && (c0 + 32 <= wb.lim_min) &&
                              !(wb.any_hole && c0 + 32 > si.hist_k && c0 < wb.hole_hi_max);
            f32x16_t pv;  // P, when it is stored
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                if constexpr (PLANES) {
                    pv[i] = score_p(s[i], sconst);
                }
                s[i] = score_ds(s[i], dp[i], sconst);
            }
            if (!full) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int jj = c0 + 8 * (i / 4) + 4 * lh + (i % 4);
                    const bool vis = (jj < lim) && !(jj >= hole_lo && jj < hole_hi);
                    float v = s[i];
                    float pe = PLANES ? pv[i] : 0.f;
                    if constexpr (HAS_MASK) {
                        v *= mw[i];
                        pe *= mw[i];
                    }
                    s[i] = vis ? v : 0.f;
                    if constexpr (PLANES) {
                        pv[i] = vis ? pe : 0.f;
                    }
                }
            }
            if constexpr (PLANES) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int key = c0 + 8 * g + 4 * lh;
                    const uint32_t off = pair_row_off + static_cast<uint32_t>(2 * c0 + 8 * g + 4 * lh) * 4u;
                    const bwd_f32x4_t wd = {s[4 * g + 0], s[4 * g + 1], s[4 * g + 2], s[4 * g + 3]};
                    const bwd_f32x4_t wp = {pv[4 * g + 0], pv[4 * g + 1], pv[4 * g + 2], pv[4 * g + 3]};
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, wd), pair_rsrc,
                                                           static_cast<int>(key < sk ? off : kOutOfRange), 0, 0);
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, wp), pair_rsrc,
                                                           static_cast<int>(key < sk ? off + 128u : kOutOfRange), 0, 0);
                }
            }
            if (want_drab) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int key = c0 + 8 * g + 4 * lh;
                    const uint32_t off = bias_row_off + static_cast<uint32_t>(key) * 4u;
                    if (bias_vec) {
                        const bwd_f32x4_t w = {s[4 * g + 0], s[4 * g + 1], s[4 * g + 2], s[4 * g + 3]};
                        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, w), drab_rsrc,
                                                               static_cast<int>(key < sk ? off : kOutOfRange), 0, 0);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float se = s[4 * g + e];  // (a copy: see the note on the dQ store below)
                            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, se), drab_rsrc,
                                                                  static_cast<int>(key + e < sk ? off + 4u * e : kOutOfRange), 0, 0);
                        }
                    }
                }
            }
            // dQ^T += K^T . dS^T: step i contracts the key pair {8 (i / 4) + i % 4, the same + 4}, one per lane half
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int vr = 8 * (i / 4) + 4 * lh + (i % 4);
#pragma unroll
                for (int mt = 0; mt < MTILES; ++mt) {
                    const int col = 32 * mt + ln;
                    const float ka = s_k[vr * D + f32_chunk_swizzle<D>(vr, col >> 2) * 4 + (col & 3)];
                    dq_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka, s[i], dq_acc[mt], 0, 0, 0);
                }
            }
        }
        __syncthreads();
    }

    // store dQ: lane holds query row (wr0 + ln), dims 32 mt + 8 g + 4 lh + 0..3
    const uint32_t row_off = static_cast<uint32_t>(wr0 + ln) * q_stride;
#pragma unroll
    for (int mt = 0; mt < MTILES; ++mt) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int d0 = 32 * mt + 8 * g + 4 * lh;
            const uint32_t off = (d0 < a.d_qk) ? row_off + d0 * 4u : kOutOfRange;
            // (__builtin_bit_cast applied to an element of a vector, v[i], reads the vector's first element whatever i
            // is: reinterpret a whole vector, or a scalar copy of the element)
            const bwd_f32x4_t w = {dq_acc[mt][4 * g + 0], dq_acc[mt][4 * g + 1], dq_acc[mt][4 * g + 2], dq_acc[mt][4 * g + 3]};
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, w), dq_rsrc, static_cast<int>(off), 0, 0);
        }
    }
}

// PLANES: P and dS are read back from what the query-tile kernel stored (see there) instead of being computed: two
// products per step instead of four, no score algebra, no rab / mask / K / V reads.
template <int D, bool HAS_RAB, bool HAS_MASK, bool PLANES = false>
__global__ __launch_bounds__(256, 1) void hstu_bwd_f32_dkv_kernel(const BwdArgs a)
{
    constexpr int BN = 32;      // query rows per LDS tile
    constexpr int CPR = D / 4;  // 16-byte chunks per row
    constexpr int TILE_FLOATS = BN * D;
    constexpr int LOADS = TILE_FLOATS / 256 / 4;
    static_assert(TILE_FLOATS % 1024 == 0, "tile must split evenly over four wavefronts");
    constexpr int QCHUNKS = D / 8;
    constexpr int MTILES = D / 32;

    __shared__ __attribute__((aligned(1024))) float s_q[TILE_FLOATS];
    __shared__ __attribute__((aligned(1024))) float s_g[TILE_FLOATS];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = uniform(tid >> 6);
    const int ln = lane & 31;
    const int lh = lane >> 5;
    const int per_level = a.n_batch * a.n_heads_k;
    const int kt_idx = blockIdx.x / per_level;
    const int rem = blockIdx.x - kt_idx * per_level;
    const int b = rem / a.n_heads_k;
    const int hk = rem - b * a.n_heads_k;
    const SeqInfo si = load_seq(a, b);
    const int sq = uniform(si.sq), sk = uniform(si.sk);
    const int c0 = kt_idx * kBlockM;
    if (c0 >= sk) {
        return;
    }
    const int cw0 = c0 + wave * 32;  // first key of this wavefront
    const int key = cw0 + ln;        // this lane's key

    const uint32_t q_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_qk * 4u;
    const uint32_t g_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_v * 4u;
    const uint32_t k_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_qk * 4u;
    const uint32_t v_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_v * 4u;
    const __amdgpu_buffer_rsrc_t k_rsrc =
        make_rsrc(static_cast<const float*>(a.k) + (si.k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_qk),
                  static_cast<uint32_t>(sk - 1) * k_stride + a.d_qk * 4u);
    const __amdgpu_buffer_rsrc_t v_rsrc =
        make_rsrc(static_cast<const float*>(a.v) + (si.k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_v),
                  static_cast<uint32_t>(sk - 1) * v_stride + a.d_v * 4u);
    const __amdgpu_buffer_rsrc_t dk_rsrc =
        make_rsrc(static_cast<float*>(a.dk) + (si.k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_qk),
                  static_cast<uint32_t>(sk - 1) * k_stride + a.d_qk * 4u);
    const __amdgpu_buffer_rsrc_t dv_rsrc =
        make_rsrc(static_cast<float*>(a.dv) + (si.k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_v),
                  static_cast<uint32_t>(sk - 1) * v_stride + a.d_v * 4u);

    // K and V fragments of this lane's key: B operands of S = Q . K^T and dP = dO . V^T (rows past sk read as zeros)
    bwd_f32x4_t kf[QCHUNKS], vf[QCHUNKS];
    {
        const uint32_t k_off = static_cast<uint32_t>(key) * k_stride;
        const uint32_t v_off = static_cast<uint32_t>(key) * v_stride;
#pragma unroll
        for (int j = 0; j < QCHUNKS; ++j) {
            const int d0 = 4 * (2 * j + lh);
            kf[j] = __builtin_bit_cast(bwd_f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(
                                                        k_rsrc, static_cast<int>(d0 < a.d_qk ? k_off + d0 * 4u : kOutOfRange), 0, 0));
            vf[j] = __builtin_bit_cast(bwd_f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(
                                                        v_rsrc, static_cast<int>(d0 < a.d_v ? v_off + d0 * 4u : kOutOfRange), 0, 0));
        }
    }
    uint32_t q_src[LOADS], g_src[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        const int slot = (wave * LOADS + i) * 64 + lane;
        const int r = slot / CPR;
        const int pc = slot - r * CPR;
        const int c = f32_chunk_swizzle<D>(r, pc);
        q_src[i] = (c * 4 < a.d_qk) ? static_cast<uint32_t>(r) * q_stride + c * 16u : kOutOfRange;
        g_src[i] = (c * 4 < a.d_v) ? static_cast<uint32_t>(r) * g_stride + c * 16u : kOutOfRange;
    }

    f32x16_t dk_acc[MTILES], dv_acc[MTILES];
#pragma unroll
    for (int mt = 0; mt < MTILES; ++mt) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            dk_acc[mt][i] = 0.f;
            dv_acc[mt][i] = 0.f;
        }
    }
    const ScoreConsts sconst = score_consts(a.alpha, a.scale);
    const uint32_t bias_bytes = static_cast<uint32_t>(a.max_q) * static_cast<uint32_t>(a.max_k) * 4u;

    // query sub-tiles that can see a key of this tile (as in the 16-bit kernel)
    const int n_qsub = (sq + 31) / 32;
    int x_first = 0;
    if (a.mask_type == 0 && !(si.n_ctx > 0 && c0 < si.hist_k)) {
        const int first_row = c0 - si.delta;
        x_first = first_row > 0 ? first_row / 32 : 0;
    }

    for (int hq = hk * a.head_ratio; hq < (hk + 1) * a.head_ratio; ++hq) {
        const __amdgpu_buffer_rsrc_t q_rsrc =
            make_rsrc(static_cast<const float*>(a.q) + (si.q0 * a.n_heads_q + hq) * static_cast<int64_t>(a.d_qk),
                      static_cast<uint32_t>(sq - 1) * q_stride + a.d_qk * 4u);
        const __amdgpu_buffer_rsrc_t g_rsrc =
            make_rsrc(static_cast<const float*>(a.grad) + (si.q0 * a.n_heads_q + hq) * static_cast<int64_t>(a.d_v),
                      static_cast<uint32_t>(sq - 1) * g_stride + a.d_v * 4u);
        const int64_t bias_plane = (static_cast<int64_t>(b) * a.n_heads_q + hq) * a.max_q * static_cast<int64_t>(a.max_k);
        const __amdgpu_buffer_rsrc_t rab_rsrc =
            make_rsrc(HAS_RAB ? static_cast<const float*>(a.rab) + bias_plane : nullptr, HAS_RAB ? bias_bytes : 0u);
        const __amdgpu_buffer_rsrc_t mask_rsrc =
            make_rsrc(HAS_MASK ? static_cast<const float*>(a.mask) + bias_plane : nullptr, HAS_MASK ? bias_bytes : 0u);
        for (int x = x_first; x < n_qsub; ++x) {
            const int rq0 = x * 32;
            const uint32_t qb = static_cast<uint32_t>(rq0) * q_stride;
            const uint32_t gb = static_cast<uint32_t>(rq0) * g_stride;
#pragma unroll
            for (int i = 0; i < LOADS; ++i) {
                __builtin_amdgcn_raw_ptr_buffer_load_lds(q_rsrc, (__attribute__((address_space(3))) void*)(s_q + (wave * LOADS + i) * 256),
                                                         16, static_cast<int>(q_src[i] + qb), 0, 0, 0);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(g_rsrc, (__attribute__((address_space(3))) void*)(s_g + (wave * LOADS + i) * 256),
                                                         16, static_cast<int>(g_src[i] + gb), 0, 0, 0);
            }
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();

            // whole block hidden from the keys of this wavefront?
            const bool active = cw0 < swept_key_limit(a, si, rq0);
            float p[16], ds[16];
            if constexpr (PLANES) {
                if (active) {
                    // only what the query-tile kernel wrote is read: the 32 x 32 blocks it swept (the blocks active
                    // here), rows of the sequence, keys ahead of its last one
                    const uint32_t pitch = 64u * static_cast<uint32_t>((a.max_k + 31) / 32);
                    const __amdgpu_buffer_rsrc_t pair_rsrc = make_rsrc(
                        static_cast<const float*>(a.p_plane) + (static_cast<int64_t>(b) * a.n_heads_q + hq) * a.max_q * static_cast<int64_t>(pitch),
                        static_cast<uint32_t>(a.max_q) * pitch * 4u);
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int r = rq0 + 8 * (i / 4) + 4 * lh + (i % 4);
                        const uint32_t off = (r < sq && key < sk)
                                                 ? (static_cast<uint32_t>(r) * pitch + static_cast<uint32_t>(2 * cw0 + ln)) * 4u
                                                 : kOutOfRange;
                        ds[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(pair_rsrc, static_cast<int>(off), 0, 0));
                        p[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                             pair_rsrc, static_cast<int>(off == kOutOfRange ? kOutOfRange : off + 128u), 0, 0));
                    }
                }
            } else if (active) {
                f32x16_t s, dp;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    s[i] = 0.f;
                    dp[i] = 0.f;
                }
                // S = Q . K^T and dP = dO . V^T: lane = key, element i = query row rq0 + 8 (i / 4) + 4 lh + i % 4
#pragma unroll
                for (int j = 0; j < QCHUNKS; ++j) {
                    const int at = ln * D + f32_chunk_swizzle<D>(ln, 2 * j + lh) * 4;
                    const bwd_f32x4_t qc = *reinterpret_cast<const bwd_f32x4_t*>(s_q + at);
                    const bwd_f32x4_t gc = *reinterpret_cast<const bwd_f32x4_t*>(s_g + at);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        s = __builtin_amdgcn_mfma_f32_32x32x2f32(qc[e], kf[j][e], s, 0, 0, 0);
                        dp = __builtin_amdgcn_mfma_f32_32x32x2f32(gc[e], vf[j][e], dp, 0, 0, 0);
                    }
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int r = rq0 + 8 * (i / 4) + 4 * lh + (i % 4);
                    float x_raw = s[i];
                    float m = 1.0f;
                    if constexpr (HAS_RAB || HAS_MASK) {
                        // lane = key: the 32 lanes of a half read 32 consecutive values of row r
                        const uint32_t off = (r < sq && key < a.max_k)
                                                 ? (static_cast<uint32_t>(r) * static_cast<uint32_t>(a.max_k) + static_cast<uint32_t>(key)) * 4u
                                                 : kOutOfRange;
                        if constexpr (HAS_RAB) {
                            x_raw += __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rab_rsrc, static_cast<int>(off), 0, 0));
                        }
                        if constexpr (HAS_MASK) {
                            m = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(mask_rsrc, static_cast<int>(off), 0, 0));
                        }
                    }
                    int lim, hole_lo, hole_hi;
                    row_bounds(si, a.mask_type, a.target_group, r, lim, hole_lo, hole_hi);
                    const bool vis = (r < sq) && (key < lim) && !(key >= hole_lo && key < hole_hi);
                    p[i] = vis ? score_p(x_raw, sconst) * m : 0.f;
                    ds[i] = vis ? score_ds(x_raw, dp[i], sconst) * m : 0.f;
                }
            }
            if (active) {
                // dV^T += dO^T . P and dK^T += Q^T . dS: step i contracts the row pair {8 (i / 4) + i % 4, the same + 4}
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int qr = 8 * (i / 4) + 4 * lh + (i % 4);
#pragma unroll
                    for (int mt = 0; mt < MTILES; ++mt) {
                        const int col = 32 * mt + ln;
                        const int at = qr * D + f32_chunk_swizzle<D>(qr, col >> 2) * 4 + (col & 3);
                        dv_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(s_g[at], p[i], dv_acc[mt], 0, 0, 0);
                        dk_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(s_q[at], ds[i], dk_acc[mt], 0, 0, 0);
                    }
                }
            }
            __syncthreads();
        }
    }

    // store dK and dV: lane holds key (cw0 + ln), dims 32 mt + 8 g + 4 lh + 0..3
    const uint32_t k_row = static_cast<uint32_t>(key) * k_stride;
    const uint32_t v_row = static_cast<uint32_t>(key) * v_stride;
#pragma unroll
    for (int mt = 0; mt < MTILES; ++mt) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int d0 = 32 * mt + 8 * g + 4 * lh;
            const bwd_f32x4_t wk = {dk_acc[mt][4 * g + 0], dk_acc[mt][4 * g + 1], dk_acc[mt][4 * g + 2], dk_acc[mt][4 * g + 3]};
            const bwd_f32x4_t wv = {dv_acc[mt][4 * g + 0], dv_acc[mt][4 * g + 1], dv_acc[mt][4 * g + 2], dv_acc[mt][4 * g + 3]};
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, wk), dk_rsrc,
                                                   static_cast<int>(d0 < a.d_qk ? k_row + d0 * 4u : kOutOfRange), 0, 0);
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, wv), dv_rsrc,
                                                   static_cast<int>(d0 < a.d_v ? v_row + d0 * 4u : kOutOfRange), 0, 0);
        }
    }
}

}  // namespace hstu
