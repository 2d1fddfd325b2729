// HSTU jagged attention backward for gfx950 (MI355X): the kernel for batches of tiny sequences -- no sequence longer
// than 32 rows or 32 keys -- at the head-dim slots 128 and 256 (the forward's counterpart: hstu_fwd_tiny_kernel.hip.h).
//
// Such a launch is bound by memory and latency: a (sequence, head) item reads 4 x 32 rows and writes 3 x 32, and its
// products are single 32 x 32 tiles.  The tuned kernels spend a 128-row workgroup per item and per launch (batch 2048,
// 2 heads, head dim 256, 32 rows: 221 us for 234 MB of operands and gradients).  Here an item is a workgroup of two
// wavefronts per (sequence, K/V head), everything in one launch, no workspace:
//   K, V -> LDS once; for each query head of the group: Q, dO -> LDS;
//   key side  (wavefront w owns keys 16 w .. + 15): S = Q K^T and dP = dO V^T with the rows as M, so that P and dS come
//             out as the B operands of dV^T += dO^T P and dK^T += Q^T dS (Q^T, dO^T by transposing LDS reads);
//   query side (wavefront w owns rows 16 w .. + 15): S^T = K Q^T, dP^T = V dO^T, dS^T, dQ^T = K^T dS^T, stored per head;
//   dK, dV stored once after the last head of the group.
// The score algebra and its rounding points are those of the tuned kernels (hstu_bwd_kernel.hip.h: P and dS rounded to
// the input type before the products that consume them; formula of
// ascendc/attention/hstu_v1/hstu_backward_v1/op_kernel/vector_score.h:159-205).  16-bit inputs, built-in mask (causal
// with context rows, target rows and target groups) or no mask, no bias.
#pragma once
#include "hstu_bwd_dq_short_kernel.hip.h"

namespace hstu {

template <typename Tag, int D>
__global__ __launch_bounds__(kTinyThreads, 1) void hstu_bwd_tiny_kernel(const BwdArgs a)
{
    static_assert(D == 128 || D == 256, "built for the head-dim slots 128 and 256");
    constexpr int TILE_ELEMS = 32 * D;
    constexpr int CPR = D / 8;
    constexpr int KSTEPS = D / 32;
    constexpr int MTILES = D / 16;
    constexpr int LOADS = TILE_ELEMS * 2 / 1024 / 2;  // 1 KiB load instructions per wavefront and tile

    __shared__ __attribute__((aligned(1024))) uint16_t s_k[TILE_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v[TILE_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_q[TILE_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_g[TILE_ELEMS];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = uniform(tid >> 6);
    const int n = lane & 15;
    const int g = lane >> 4;

    zero_tail_rows(a.dq, a.offs_q, a.n_batch, a.idx64, a.total_q, static_cast<int64_t>(a.n_heads_q) * a.d_qk, kTinyThreads);
    zero_tail_rows(a.dk, a.offs_k, a.n_batch, a.idx64, a.total_k, static_cast<int64_t>(a.n_heads_k) * a.d_qk, kTinyThreads);
    zero_tail_rows(a.dv, a.offs_k, a.n_batch, a.idx64, a.total_k, static_cast<int64_t>(a.n_heads_k) * a.d_v, kTinyThreads);

    // ---- the item of this workgroup: (sequence, K/V head) ----
    const int item = static_cast<int>(blockIdx.x);
    if (item >= a.n_batch * a.n_heads_k) {
        return;
    }
    const int b = div_small(item, a.n_heads_k);
    const int hk = item - b * a.n_heads_k;
    const SeqInfo si = load_seq(a, b);  // (the host sends a launch here only when no sequence passes kTinyRows rows or keys)
    const int sq = si.sq, sk = si.sk;

    const uint32_t q_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_qk * 2u;
    const uint32_t g_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_v * 2u;
    const uint32_t k_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_qk * 2u;
    const uint32_t v_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_v * 2u;
    const u32x4_t k_rsrc =
        make_rsrc_words(static_cast<const uint8_t*>(a.k) + (si.k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_qk) * 2,
                        sk > 0 ? static_cast<uint32_t>(sk - 1) * k_stride + a.d_qk * 2u : 0u);
    const u32x4_t v_rsrc =
        make_rsrc_words(static_cast<const uint8_t*>(a.v) + (si.k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_v) * 2,
                        sk > 0 ? static_cast<uint32_t>(sk - 1) * v_stride + a.d_v * 2u : 0u);

    // ---- tile loads: instruction i of a tile fills its bytes [1024 i, + 1024); piece 64 i + lane is row piece / CPR,
    // physical chunk piece % CPR, which holds the logical chunk the swizzle names.  Rows past the sequence read as zeros.
    auto load_tile = [&](u32x4_t rsrc, uint16_t* tile, uint32_t stride, int dims) {
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const int instr = 2 * i + wave;
            const int piece = instr * 64 + lane;
            const int r = piece / CPR;
            const int cs = both_ways16_swizzle<D>(r, piece % CPR);
            const uint32_t src = (cs * 8 < dims) ? static_cast<uint32_t>(r) * stride + cs * 16u : kOutOfRange;
            request_to_lds_b128(rsrc, lds_address(tile) + instr * 1024u, src);
        }
    };
    load_tile(k_rsrc, s_k, k_stride, a.d_qk);
    load_tile(v_rsrc, s_v, v_stride, a.d_v);

    // LDS read offsets relative to a tile, in elements: plain read of row n (+ 16), MFMA step js; transposed read of rows
    // 4 g .. 4 g + 3 (+ 16), dims 16 mt .. + 15
    int n_lane_off[KSTEPS];
#pragma unroll
    for (int js = 0; js < KSTEPS; ++js) {
        n_lane_off[js] = n * D + both_ways16_swizzle<D>(n, 4 * js + g) * 8;
    }
    const int vr = 4 * g + (n >> 2);
    const int t_row_off = vr * D + 4 * (n & 1);
    const int t_chunk_lo = (n & 3) >> 1;
    auto t_lane_off = [&](int mt) -> int { return t_row_off + both_ways16_swizzle<D>(vr, 2 * mt + t_chunk_lo) * 8; };
    auto read_t = [&](const uint16_t* tile, int mt) -> u32x4_t {
        const uint16_t* const p = tile + t_lane_off(mt);
        const u32x2_t lo = lds_read_tr16_b64(p);
        const u32x2_t hi = lds_read_tr16_b64(p + 16 * D);
        const u32x4_t r = {lo[0], lo[1], hi[0], hi[1]};
        return r;
    };

    const ScoreConsts sconst = score_consts(a.alpha, a.scale);
    // Visibility under the built-in mask (or of everything inside the sequence), the same for every head: lane l works out
    // the bounds of row l mod 32 once, the lanes that need them fetch them, and what stays is one bit per accumulator
    // element: bit e of key_side for (row 16 (e / 4) + 4 g + e % 4, key 16 w + n), of query_side for (row 16 w + n, key
    // 16 (e / 4) + 4 g + e % 4).
    uint32_t key_side = 0, query_side = 0;
    {
        int lim, hole_lo, hole_hi;
        row_bounds(si, a.mask_type, a.target_group, lane & 31, lim, hole_lo, hole_hi);
        lim = (lane & 31) < sq ? lim : 0;
        const int mine = lim | (hole_lo << 8) | (hole_hi << 16);  // (each at most 32)
        auto sees = [](int bounds, int key) -> bool {
            return key < (bounds & 255) && !(key >= ((bounds >> 8) & 255) && key < (bounds >> 16));
        };
        const int of_my_row = __shfl(mine, 16 * wave + n);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int other = 16 * (e / 4) + 4 * g + (e % 4);
            key_side |= (sees(__shfl(mine, other), 16 * wave + n) ? 1u : 0u) << e;
            query_side |= (sees(of_my_row, other) ? 1u : 0u) << e;
        }
    }

    f32x4_t dk_acc[MTILES], dv_acc[MTILES];
#pragma unroll
    for (int mt = 0; mt < MTILES; ++mt) {
        dk_acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        dv_acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }

    for (int r = 0; r < a.head_ratio; ++r) {
        const int h = hk * a.head_ratio + r;
        const u32x4_t q_rsrc = make_rsrc_words(
            static_cast<const uint8_t*>(a.q) + (si.q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_qk) * 2,
            sq > 0 ? static_cast<uint32_t>(sq - 1) * q_stride + a.d_qk * 2u : 0u);
        const u32x4_t g_rsrc = make_rsrc_words(
            static_cast<const uint8_t*>(a.grad) + (si.q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_v) * 2,
            sq > 0 ? static_cast<uint32_t>(sq - 1) * g_stride + a.d_v * 2u : 0u);
        load_tile(q_rsrc, s_q, q_stride, a.d_qk);
        load_tile(g_rsrc, s_g, g_stride, a.d_v);
        // everything asked for is in (mine, then everybody's)
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt((0 & 15) | (7 << 4) | (15 << 8));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);

        // ---- key side: S (32 rows x 16 keys) = Q . K^T, dP = dO . V^T; lane (n, g) holds rows 16 j + 4 g + r of key 16 w + n
        {
            f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
            f32x4_t dp0 = {0.f, 0.f, 0.f, 0.f}, dp1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int js = 0; js < KSTEPS; ++js) {
                const u32x4_t kf = *reinterpret_cast<const u32x4_t*>(s_k + n_lane_off[js] + 16 * wave * D);
                const u32x4_t vf = *reinterpret_cast<const u32x4_t*>(s_v + n_lane_off[js] + 16 * wave * D);
                const u32x4_t qa = *reinterpret_cast<const u32x4_t*>(s_q + n_lane_off[js]);
                const u32x4_t qb = *reinterpret_cast<const u32x4_t*>(s_q + n_lane_off[js] + 16 * D);
                s0 = mfma16<Tag>(qa, kf, s0);
                s1 = mfma16<Tag>(qb, kf, s1);
                const u32x4_t ga = *reinterpret_cast<const u32x4_t*>(s_g + n_lane_off[js]);
                const u32x4_t gb = *reinterpret_cast<const u32x4_t*>(s_g + n_lane_off[js] + 16 * D);
                dp0 = mfma16<Tag>(ga, vf, dp0);
                dp1 = mfma16<Tag>(gb, vf, dp1);
            }
            float ds[8], pv[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float sv = e < 4 ? s0[e] : s1[e - 4];
                const float dv = e < 4 ? dp0[e] : dp1[e - 4];
                const bool vis = (key_side >> e) & 1u;
                ds[e] = vis ? score_ds(sv, dv, sconst) : 0.f;
                pv[e] = vis ? score_p(sv, sconst) : 0.f;
            }
            const u32x4_t db = {pack2<Tag>(ds[0], ds[1]), pack2<Tag>(ds[2], ds[3]), pack2<Tag>(ds[4], ds[5]), pack2<Tag>(ds[6], ds[7])};
            const u32x4_t pb = {pack2<Tag>(pv[0], pv[1]), pack2<Tag>(pv[2], pv[3]), pack2<Tag>(pv[4], pv[5]), pack2<Tag>(pv[6], pv[7])};
            // dV^T (D dims x 16 keys) += dO^T . P, dK^T += Q^T . dS (contraction over the 32 rows)
#pragma unroll
            for (int mt = 0; mt < MTILES; ++mt) {
                dv_acc[mt] = mfma16<Tag>(read_t(s_g, mt), pb, dv_acc[mt]);
                dk_acc[mt] = mfma16<Tag>(read_t(s_q, mt), db, dk_acc[mt]);
            }
        }

        // ---- query side: S^T (32 keys x 16 rows) = K . Q^T, dP^T = V . dO^T; lane (n, g) holds keys 16 j + 4 g + r of row 16 w + n
        f32x4_t dq_acc[MTILES];
        {
            f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
            f32x4_t dp0 = {0.f, 0.f, 0.f, 0.f}, dp1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int js = 0; js < KSTEPS; ++js) {
                const u32x4_t qf = *reinterpret_cast<const u32x4_t*>(s_q + n_lane_off[js] + 16 * wave * D);
                const u32x4_t gf = *reinterpret_cast<const u32x4_t*>(s_g + n_lane_off[js] + 16 * wave * D);
                const u32x4_t ka = *reinterpret_cast<const u32x4_t*>(s_k + n_lane_off[js]);
                const u32x4_t kb = *reinterpret_cast<const u32x4_t*>(s_k + n_lane_off[js] + 16 * D);
                s0 = mfma16<Tag>(ka, qf, s0);
                s1 = mfma16<Tag>(kb, qf, s1);
                const u32x4_t va = *reinterpret_cast<const u32x4_t*>(s_v + n_lane_off[js]);
                const u32x4_t vb = *reinterpret_cast<const u32x4_t*>(s_v + n_lane_off[js] + 16 * D);
                dp0 = mfma16<Tag>(va, gf, dp0);
                dp1 = mfma16<Tag>(vb, gf, dp1);
            }
            float ds[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float sv = e < 4 ? s0[e] : s1[e - 4];
                const float dv = e < 4 ? dp0[e] : dp1[e - 4];
                const bool vis = (query_side >> e) & 1u;
                ds[e] = vis ? score_ds(sv, dv, sconst) : 0.f;
            }
            const u32x4_t db = {pack2<Tag>(ds[0], ds[1]), pack2<Tag>(ds[2], ds[3]), pack2<Tag>(ds[4], ds[5]), pack2<Tag>(ds[6], ds[7])};
#pragma unroll
            for (int mt = 0; mt < MTILES; ++mt) {
                dq_acc[mt] = mfma16<Tag>(read_t(s_k, mt), db, f32x4_t{0.f, 0.f, 0.f, 0.f});
            }
        }
        // ---- store dQ of this head: lane (n, g) holds dims 16 mt + 4 g + 0..3 of row 16 w + n; through the Q tile (nobody
        // reads it any more once both wavefronts are here), whole lines per store instruction ----
        __syncthreads();
        if (sq > 0) {
            const __amdgpu_buffer_rsrc_t dq_rsrc =
                make_rsrc(static_cast<uint8_t*>(a.dq) + (si.q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_qk) * 2,
                          static_cast<uint32_t>(sq - 1) * q_stride + a.d_qk * 2u);
            uint16_t* const stage = s_q + wave * (16 * D);
#pragma unroll
            for (int mt = 0; mt < MTILES; ++mt) {
                u32x2_t w;
                w[0] = pack2<Tag>(dq_acc[mt][0], dq_acc[mt][1]);
                w[1] = pack2<Tag>(dq_acc[mt][2], dq_acc[mt][3]);
                const int chunk = (2 * mt + (g >> 1)) ^ n;
                *reinterpret_cast<u32x2_t*>(stage + n * D + chunk * 8 + 4 * (g & 1)) = w;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            constexpr int RPI = 64 / CPR;
            const int rr = lane / CPR;
            const int cc = lane % CPR;
#pragma unroll
            for (int i = 0; i < kShortWaveM / RPI; ++i) {
                const int row = i * RPI + rr;
                const u32x4_t piece = *reinterpret_cast<const u32x4_t*>(stage + row * D + (cc ^ row) * 8);
                const uint32_t off = (cc * 8 < a.d_qk) ? static_cast<uint32_t>(16 * wave + row) * q_stride + cc * 16u : kOutOfRange;
                __builtin_amdgcn_raw_buffer_store_b128(piece, dq_rsrc, static_cast<int>(off), 0, 2);
            }
        }
        // (the stage is read before the next head's Q rows are asked for into it)
        __syncthreads();
    }

    // ---- store dK and dV: lane (n, g) holds dims 16 mt + 4 g + 0..3 of key 16 w + n; through the K and V tiles ----
    auto store_keys = [&](uint16_t* tile, const f32x4_t (&acc)[MTILES], void* out, uint32_t stride, int dims) {
        const __amdgpu_buffer_rsrc_t rsrc =
            make_rsrc(static_cast<uint8_t*>(out) + (si.k0 * a.n_heads_k + hk) * static_cast<int64_t>(dims) * 2,
                      static_cast<uint32_t>(sk - 1) * stride + static_cast<uint32_t>(dims) * 2u);
        uint16_t* const stage = tile + wave * (16 * D);
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
            u32x2_t w;
            w[0] = pack2<Tag>(acc[mt][0], acc[mt][1]);
            w[1] = pack2<Tag>(acc[mt][2], acc[mt][3]);
            const int chunk = (2 * mt + (g >> 1)) ^ n;
            *reinterpret_cast<u32x2_t*>(stage + n * D + chunk * 8 + 4 * (g & 1)) = w;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        constexpr int RPI = 64 / CPR;
        const int rr = lane / CPR;
        const int cc = lane % CPR;
#pragma unroll
        for (int i = 0; i < kShortWaveM / RPI; ++i) {
            const int row = i * RPI + rr;
            const u32x4_t piece = *reinterpret_cast<const u32x4_t*>(stage + row * D + (cc ^ row) * 8);
            const uint32_t off = (cc * 8 < dims) ? static_cast<uint32_t>(16 * wave + row) * stride + cc * 16u : kOutOfRange;
            __builtin_amdgcn_raw_buffer_store_b128(piece, rsrc, static_cast<int>(off), 0, 2);
        }
    };
    // (the last head's barrier has passed: nobody reads the K / V tiles any more)
    if (sk > 0) {
        store_keys(s_k, dk_acc, a.dk, k_stride, a.d_qk);
        store_keys(s_v, dv_acc, a.dv, v_stride, a.d_v);
    }
}

}  // namespace hstu
