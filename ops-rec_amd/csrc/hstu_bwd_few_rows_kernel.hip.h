// HSTU jagged attention backward for gfx950 (MI355X): the kernel for sequences of few query rows -- at most 64 -- against
// keys of any length (candidates attending to a long history), head dims up to 128, one K/V head per query head.
//
// The tuned kernels give such a sequence one 128-row query tile, mostly empty, and a pair of workgroups per 128 keys,
// each of which starts up (offsets, Q and dO rows) for a sweep of one or two steps: batch 2048 x 4 heads x 52 rows x
// 1000 keys at head dim 64 takes 2.09 ms, 1.64 of them in 131 072 key-tile workgroups, and K and V are read twice.
// Here a workgroup of four wavefronts owns a (sequence, head) whole: Q and dO stay in LDS, K and V stream through a
// ring of 32-key sub-tiles exactly once, and each step finishes its 32 keys:
//   query side (wavefront w owns rows 16 w .. + 15): S^T = K Q^T, dP^T = V dO^T, P and dS (masked, rounded to the input
//              type) into an LDS exchange buffer, dQ^T += K^T dS^T;
//   key side   (wavefront w owns keys 16 (w & 1) .. + 15 of the step; w < 2: dV^T = dO^T P, w >= 2: dK^T = Q^T dS, the
//              contraction over all 64 rows), stored straight away: no accumulation across workgroups, no workspace.
// Five products per pair, one launch.  The score algebra and its rounding points are those of the tuned kernels
// (hstu_bwd_kernel.hip.h; formula of ascendc/attention/hstu_v1/hstu_backward_v1/op_kernel/vector_score.h:159-205).
// 16-bit inputs, built-in mask (causal with context rows, target rows and target groups) or no mask, no bias.
#pragma once
#include "hstu_bwd_dq_short_kernel.hip.h"

namespace hstu {

// LDS layout of a tile with rows of 64 elements (eight 16-byte chunks) that is free of bank conflicts for the plain
// read of 16 consecutive rows, one chunk each, and for the transposing read of rows 4 g .. 4 g + 3 (found by search
// over the linear maps of the row bits; adding 16 or 32 to the row leaves the term alone)
__device__ __forceinline__ int both_ways16_swizzle64(int row, int chunk)
{
    const int b1 = (row >> 1) & 1, b2 = (row >> 2) & 1, b3 = (row >> 3) & 1;
    return chunk ^ (b1 | (b2 << 1) | ((b1 ^ b3) << 2));
}
// the layout of the kernel's tiles by head-dim slot (rows of 128 elements: that of the query-tile kernel for short rows)
template <int D>
__device__ __forceinline__ int few_rows_swizzle(int row, int chunk)
{
    static_assert(D == 64 || D == 128, "head-dim slots 64 and 128");
    if constexpr (D == 64) {
        return both_ways16_swizzle64(row, chunk);
    } else {
        return both_ways16_swizzle<D>(row, chunk);
    }
}
// The exchange buffer [64 rows][32 keys] in 8-byte chunks (4 keys): the query side writes a row's chunks g and 4 + g,
// the key side reads 4-row x 16-key blocks transposing
__device__ __forceinline__ int exchange_chunk(int row, int chunk) { return chunk ^ ((((row >> 2) & 1) << 2) | (((row >> 3) & 1) << 1)); }

template <typename Tag, int D>
__global__ __launch_bounds__(kFewRowsThreads, 2) void hstu_bwd_few_rows_kernel(const BwdArgs a)
{
    static_assert(D == 64 || D == 128, "built for the head-dim slots 64 and 128");
    constexpr int ROWS = kFewRows;
    constexpr int SUB_ELEMS = 32 * D;
    constexpr int CPR = D / 8;
    constexpr int KSTEPS = D / 32;
    constexpr int MTILES = D / 16;
    constexpr int NSTAGE = D == 64 ? 3 : 2;  // (72 KiB of LDS at the slot 128: two workgroups per CU)
    constexpr int LPW = SUB_ELEMS * 2 / 1024 / 4;      // 1 KiB load instructions per wavefront and sub-tile (K, and again V)
    constexpr int QLOADS = ROWS * D * 2 / 1024 / 4;    // ... per wavefront for the Q tile (and again dO)
    constexpr int STORES = MTILES / 2;                 // store instructions per wavefront and step (dV or dK of 16 keys)
    static_assert(LPW >= 1 && QLOADS >= 1, "whole load instructions per wavefront");
    // at the top of step x its sub-tile has landed when nothing older than this is open: the requests of the steps after
    // it and the stores of the steps since it was asked for (vector memory operations complete in the order of issue)
    constexpr int kOpen = (NSTAGE - 2) * 2 * LPW + (NSTAGE - 1) * STORES;
    static_assert(kOpen < 64, "6 bits of count");
    constexpr int kWaitStage = (kOpen & 15) | (7 << 4) | (15 << 8) | ((kOpen >> 4) << 14);
    constexpr uint32_t kPastEnd = 0x40000000u;

    __shared__ __attribute__((aligned(1024))) uint16_t s_q[ROWS * D];
    __shared__ __attribute__((aligned(1024))) uint16_t s_g[ROWS * D];
    __shared__ __attribute__((aligned(1024))) uint16_t s_k[NSTAGE][SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v[NSTAGE][SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_p[ROWS * 32];
    __shared__ __attribute__((aligned(1024))) uint16_t s_ds[ROWS * 32];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = uniform(tid >> 6);
    const int n = lane & 15;
    const int g = lane >> 4;

    zero_tail_rows(a.dq, a.offs_q, a.n_batch, a.idx64, a.total_q, static_cast<int64_t>(a.n_heads_q) * a.d_qk, kFewRowsThreads);
    zero_tail_rows(a.dk, a.offs_k, a.n_batch, a.idx64, a.total_k, static_cast<int64_t>(a.n_heads_k) * a.d_qk, kFewRowsThreads);
    zero_tail_rows(a.dv, a.offs_k, a.n_batch, a.idx64, a.total_k, static_cast<int64_t>(a.n_heads_k) * a.d_v, kFewRowsThreads);

    // ---- the item of this workgroup: (sequence, head) ----
    const int item = static_cast<int>(blockIdx.x);
    if (item >= a.n_batch * a.n_heads_k) {
        return;
    }
    const int b = div_small(item, a.n_heads_k);
    const int h = item - b * a.n_heads_k;
    const SeqInfo si = load_seq(a, b);  // (the host sends a launch here only when no sequence passes kFewRows query rows)
    const int sq = si.sq, sk = si.sk;
    const int wr0 = wave * kShortWaveM;

    const uint32_t q_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_qk * 2u;
    const uint32_t g_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_v * 2u;
    const uint32_t k_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_qk * 2u;
    const uint32_t v_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_v * 2u;
    const uint32_t k_bytes = sk > 0 ? static_cast<uint32_t>(sk - 1) * k_stride + a.d_qk * 2u : 0u;
    const uint32_t v_bytes = sk > 0 ? static_cast<uint32_t>(sk - 1) * v_stride + a.d_v * 2u : 0u;
    const uint32_t q_bytes = sq > 0 ? static_cast<uint32_t>(sq - 1) * q_stride + a.d_qk * 2u : 0u;
    const uint32_t g_bytes = sq > 0 ? static_cast<uint32_t>(sq - 1) * g_stride + a.d_v * 2u : 0u;
    const int64_t k_first = (si.k0 * a.n_heads_k + h) * static_cast<int64_t>(a.d_qk) * 2;
    const int64_t v_first = (si.k0 * a.n_heads_k + h) * static_cast<int64_t>(a.d_v) * 2;
    const int64_t q_first = (si.q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_qk) * 2;
    const int64_t g_first = (si.q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_v) * 2;
    const u32x4_t k_rsrc = make_rsrc_words(static_cast<const uint8_t*>(a.k) + k_first, k_bytes);
    const u32x4_t v_rsrc = make_rsrc_words(static_cast<const uint8_t*>(a.v) + v_first, v_bytes);
    const u32x4_t q_rsrc = make_rsrc_words(static_cast<const uint8_t*>(a.q) + q_first, q_bytes);
    const u32x4_t g_rsrc = make_rsrc_words(static_cast<const uint8_t*>(a.grad) + g_first, g_bytes);
    const __amdgpu_buffer_rsrc_t dk_rsrc = make_rsrc(static_cast<uint8_t*>(a.dk) + k_first, k_bytes);
    const __amdgpu_buffer_rsrc_t dv_rsrc = make_rsrc(static_cast<uint8_t*>(a.dv) + v_first, v_bytes);

    // ---- Q and dO: piece 64 i + lane of a tile is row piece / CPR, physical chunk piece % CPR, which holds the logical
    // chunk the swizzle names; rows past the sequence and dims past the head dim read as zeros ----
#pragma unroll
    for (int i = 0; i < QLOADS; ++i) {
        const int instr = wave * QLOADS + i;
        const int piece = instr * 64 + lane;
        const int r = piece / CPR;
        const int cs = few_rows_swizzle<D>(r, piece % CPR);
        request_to_lds_b128(q_rsrc, lds_address(s_q) + instr * 1024u,
                            (cs * 8 < a.d_qk) ? static_cast<uint32_t>(r) * q_stride + cs * 16u : kOutOfRange);
        request_to_lds_b128(g_rsrc, lds_address(s_g) + instr * 1024u,
                            (cs * 8 < a.d_v) ? static_cast<uint32_t>(r) * g_stride + cs * 16u : kOutOfRange);
    }
    // per-lane source offsets of the sub-tile loads
    uint32_t k_src[LPW], v_src[LPW];
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
        const int piece = (wave * LPW + i) * 64 + lane;
        const int r = piece / CPR;
        const int cs = few_rows_swizzle<D>(r, piece % CPR);
        k_src[i] = (cs * 8 < a.d_qk) ? static_cast<uint32_t>(r) * k_stride + cs * 16u : kOutOfRange;
        v_src[i] = (cs * 8 < a.d_v) ? static_cast<uint32_t>(r) * v_stride + cs * 16u : kOutOfRange;
    }
    // every row of a sequence sees keys up to its last row's limit, which is the last key: all 32-key blocks are swept
    const int n_sub = sq > 0 ? (sk + 31) / 32 : 0;
    auto request = [&](int stage, int x) {
        const uint32_t past = x < n_sub ? 0u : kPastEnd;
        const uint32_t kb = static_cast<uint32_t>(x * 32) * k_stride + past;
        const uint32_t vb = static_cast<uint32_t>(x * 32) * v_stride + past;
#pragma unroll
        for (int i = 0; i < LPW; ++i) {
            request_to_lds_b128(k_rsrc, lds_address(s_k[stage]) + (wave * LPW + i) * 1024u, k_src[i] + kb);
            request_to_lds_b128(v_rsrc, lds_address(s_v[stage]) + (wave * LPW + i) * 1024u, v_src[i] + vb);
        }
    };
#pragma unroll
    for (int i = 0; i < NSTAGE - 1; ++i) {
        request(i, i);
    }

    // LDS read offsets relative to a tile, in elements: plain read of row n (+ 16), MFMA step js; transposed read of rows
    // 4 g .. 4 g + 3 (+ 16), dims 16 mt .. + 15
    int n_lane_off[KSTEPS];
#pragma unroll
    for (int js = 0; js < KSTEPS; ++js) {
        n_lane_off[js] = n * D + few_rows_swizzle<D>(n, 4 * js + g) * 8;
    }
    const int vr = 4 * g + (n >> 2);
    const int t_row_off = vr * D + 4 * (n & 1);
    const int t_chunk_lo = (n & 3) >> 1;
    auto read_t = [&](const uint16_t* tile, int mt) -> u32x4_t {
        const uint16_t* const p = tile + t_row_off + few_rows_swizzle<D>(vr, 2 * mt + t_chunk_lo) * 8;
        const u32x2_t lo = lds_read_tr16_b64(p);
        const u32x2_t hi = lds_read_tr16_b64(p + 16 * D);
        const u32x4_t r = {lo[0], lo[1], hi[0], hi[1]};
        return r;
    };
    // exchange buffer: what this lane writes (row wr0 + n: keys 4 g .. + 3 and 16 + 4 g .. + 3 of the step), in elements ...
    const int x_row = wr0 + n;
    const int x_write_lo = x_row * 32 + exchange_chunk(x_row, g) * 4;
    const int x_write_hi = x_row * 32 + exchange_chunk(x_row, 4 + g) * 4;
    // ... and reads as the B operand of a key-side product: rows 4 g + (n >> 2) (+ 16, + 32, + 48), keys 16 kh + 4 (n & 3) .. + 3
    const int kh = wave & 1;
    const bool dk_role = wave >= 2;
    const int x_read = vr * 32 + exchange_chunk(vr, 4 * kh + (n & 3)) * 4;  // (+ 16 rows: the same chunk; + 32, + 48 likewise)

    // visibility of this lane's row (clamped into the sequence: rows past it hold zeros and produce zeros)
    int row = wr0 + n;
    row = row < sq - 1 ? row : sq - 1;
    int lim, hole_lo, hole_hi;
    row_bounds(si, a.mask_type, a.target_group, row, lim, hole_lo, hole_hi);
    const WaveBounds wb = wave_bounds(a.mask_type, wr0, sq, sk, si.n_ctx, si.n_tgt, a.target_group, wr0 < sq, kShortWaveM);
    const int lim_lane = lim - 4 * g;
    const int hole_lo_lane = hole_lo - 4 * g;
    const int hole_hi_lane = hole_hi - 4 * g;

    const ScoreConsts sconst = score_consts(a.alpha, a.scale);
    f32x4_t dq_acc[MTILES];
#pragma unroll
    for (int mt = 0; mt < MTILES; ++mt) {
        dq_acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }

    // Q, dO and the first sub-tiles are in (mine, then everybody's) before anybody reads them
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt((0 & 15) | (7 << 4) | (15 << 8));
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    // the rows of this wavefront as B operands
    u32x4_t qf[KSTEPS], gf[KSTEPS];
#pragma unroll
    for (int js = 0; js < KSTEPS; ++js) {
        qf[js] = *reinterpret_cast<const u32x4_t*>(s_q + wr0 * D + n_lane_off[js]);
        gf[js] = *reinterpret_cast<const u32x4_t*>(s_g + wr0 * D + n_lane_off[js]);
    }

    int stage = 0;
    for (int x = 0; x < n_sub; ++x) {
        // sub-tile x has landed (mine, then everybody's); nobody reads the stage of step x - 1 or the exchange buffer any more
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(kWaitStage);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        const int ahead = stage >= 1 ? stage - 1 : NSTAGE - 1;  // (x + NSTAGE - 1) mod NSTAGE
        request(ahead, x + NSTAGE - 1);
        const uint16_t* const kn = s_k[stage];
        const uint16_t* const vn = s_v[stage];
        const int c0 = x * 32;

        // ---- query side: S^T = K Q^T and dP^T = V dO^T (32 keys x 16 rows each, two blocks of 16 keys) ----
        f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = s0, dp0 = s0, dp1 = s0;
#pragma unroll
        for (int js = 0; js < KSTEPS; ++js) {
            const u32x4_t ka = *reinterpret_cast<const u32x4_t*>(kn + n_lane_off[js]);
            const u32x4_t kb = *reinterpret_cast<const u32x4_t*>(kn + n_lane_off[js] + 16 * D);
            s0 = mfma16<Tag>(ka, qf[js], s0);
            s1 = mfma16<Tag>(kb, qf[js], s1);
            const u32x4_t va = *reinterpret_cast<const u32x4_t*>(vn + n_lane_off[js]);
            const u32x4_t vb = *reinterpret_cast<const u32x4_t*>(vn + n_lane_off[js] + 16 * D);
            dp0 = mfma16<Tag>(va, gf[js], dp0);
            dp1 = mfma16<Tag>(vb, gf[js], dp1);
        }
        // element (j, r) is key c0 + 16 j + 4 g + r of this lane's row
        float ds[8], pv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float sv = e < 4 ? s0[e] : s1[e - 4];
            const float dv = e < 4 ? dp0[e] : dp1[e - 4];
            ds[e] = score_ds(sv, dv, sconst);
            pv[e] = score_p(sv, sconst);
        }
        const bool full = (c0 + 32 <= wb.lim_min) && !(wb.any_hole && c0 + 32 > si.hist_k && c0 < wb.hole_hi_max);
        if (!full) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int kk = c0 + 16 * (e / 4) + (e % 4);  // + 4 g is folded into the *_lane bounds
                const bool vis = (kk < lim_lane) && !(kk >= hole_lo_lane && kk < hole_hi_lane);
                ds[e] = vis ? ds[e] : 0.f;
                pv[e] = vis ? pv[e] : 0.f;
            }
        }
        const u32x4_t db = {pack2<Tag>(ds[0], ds[1]), pack2<Tag>(ds[2], ds[3]), pack2<Tag>(ds[4], ds[5]), pack2<Tag>(ds[6], ds[7])};
        {
            const u32x2_t d_lo = {db[0], db[1]}, d_hi = {db[2], db[3]};
            const u32x2_t p_lo = {pack2<Tag>(pv[0], pv[1]), pack2<Tag>(pv[2], pv[3])};
            const u32x2_t p_hi = {pack2<Tag>(pv[4], pv[5]), pack2<Tag>(pv[6], pv[7])};
            *reinterpret_cast<u32x2_t*>(s_ds + x_write_lo) = d_lo;
            *reinterpret_cast<u32x2_t*>(s_ds + x_write_hi) = d_hi;
            *reinterpret_cast<u32x2_t*>(s_p + x_write_lo) = p_lo;
            *reinterpret_cast<u32x2_t*>(s_p + x_write_hi) = p_hi;
        }
        // dQ^T (D dims x 16 rows) += K^T dS^T
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
            dq_acc[mt] = mfma16<Tag>(read_t(kn, mt), db, dq_acc[mt]);
        }
        // P and dS of all 64 rows are in the exchange buffer
        __syncthreads();

        // ---- key side: dV^T (D dims x 16 keys) = dO^T P, or dK^T = Q^T dS, over the 64 rows; stored at once ----
        {
            const uint16_t* const xs = (dk_role ? s_ds : s_p) + x_read;
            const uint16_t* const rows = dk_role ? s_q : s_g;
            u32x4_t bop[ROWS / 32];
#pragma unroll
            for (int ks = 0; ks < ROWS / 32; ++ks) {
                const u32x2_t lo = lds_read_tr16_b64(xs + ks * 32 * 32);
                const u32x2_t hi = lds_read_tr16_b64(xs + ks * 32 * 32 + 16 * 32);
                bop[ks] = u32x4_t{lo[0], lo[1], hi[0], hi[1]};
            }
            typedef __attribute__((ext_vector_type(2))) unsigned u2_t;
            const __amdgpu_buffer_rsrc_t out_rsrc = dk_role ? dk_rsrc : dv_rsrc;
            const uint32_t out_stride = dk_role ? k_stride : v_stride;
            const int out_dims = dk_role ? a.d_qk : a.d_v;
            const uint32_t row_off = static_cast<uint32_t>(c0 + 16 * kh + n) * out_stride;
#pragma unroll
            for (int mt = 0; mt < MTILES; mt += 2) {
                f32x4_t acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = acc0;
#pragma unroll
                for (int ks = 0; ks < ROWS / 32; ++ks) {
                    acc0 = mfma16<Tag>(read_t(rows + ks * 32 * D, mt), bop[ks], acc0);
                    acc1 = mfma16<Tag>(read_t(rows + ks * 32 * D, mt + 1), bop[ks], acc1);
                }
                // lane (n, g) holds dims 16 mt + 4 g + 0..3 of key c0 + 16 kh + n for both tiles; lanes 16 apart trade one
                // of them (v_permlane16_swap: odd rows of the first operand against even rows of the second), after which
                // a lane holds 8 dims in a row: of tile mt at 8 (g / 2) when g is even, of tile mt + 1 when it is odd
                // (keys past the sequence fall outside the descriptor)
                const u2_t lo = __builtin_amdgcn_permlane16_swap(pack2<Tag>(acc0[0], acc0[1]), pack2<Tag>(acc1[0], acc1[1]), false, false);
                const u2_t hi = __builtin_amdgcn_permlane16_swap(pack2<Tag>(acc0[2], acc0[3]), pack2<Tag>(acc1[2], acc1[3]), false, false);
                const u32x4_t piece = {lo[0], hi[0], lo[1], hi[1]};
                const int d0 = 16 * (mt + (g & 1)) + 8 * (g >> 1);
                __builtin_amdgcn_raw_buffer_store_b128(piece, out_rsrc, static_cast<int>(d0 < out_dims ? row_off + d0 * 2u : kOutOfRange), 0, 0);
            }
        }
        stage = stage + 1 < NSTAGE ? stage + 1 : 0;
    }

    // ---- a sequence without query rows: its keys get zeros ----
    if (n_sub == 0 && sk > 0) {
        const u32x4_t zero = {0u, 0u, 0u, 0u};
        const int k_pieces = a.d_qk / 8, v_pieces = a.d_v / 8;
        for (int i = tid; i < sk * k_pieces; i += kFewRowsThreads) {
            const int r = i / k_pieces;
            __builtin_amdgcn_raw_buffer_store_b128(zero, dk_rsrc, static_cast<int>(r * k_stride + (i - r * k_pieces) * 16u), 0, 0);
        }
        for (int i = tid; i < sk * v_pieces; i += kFewRowsThreads) {
            const int r = i / v_pieces;
            __builtin_amdgcn_raw_buffer_store_b128(zero, dv_rsrc, static_cast<int>(r * v_stride + (i - r * v_pieces) * 16u), 0, 0);
        }
    }

    // ---- store dQ: lane (n, g) holds dims 16 mt + 4 g + 0..3 of row wr0 + n; through the Q tile (nobody reads it any
    // more once every wavefront is here, and every request has landed), whole lines per store instruction ----
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (sq > 0) {
        const __amdgpu_buffer_rsrc_t dq_rsrc = make_rsrc(static_cast<uint8_t*>(a.dq) + q_first, q_bytes);
        uint16_t* const stage_rows = s_q + wave * (16 * D);
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
            u32x2_t w;
            w[0] = pack2<Tag>(dq_acc[mt][0], dq_acc[mt][1]);
            w[1] = pack2<Tag>(dq_acc[mt][2], dq_acc[mt][3]);
            const int chunk = (2 * mt + (g >> 1)) ^ (n & (CPR - 1));
            *reinterpret_cast<u32x2_t*>(stage_rows + n * D + chunk * 8 + 4 * (g & 1)) = w;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        constexpr int RPI = 64 / CPR;
        const int rr = lane / CPR;
        const int cc = lane % CPR;
#pragma unroll
        for (int i = 0; i < kShortWaveM / RPI; ++i) {
            const int r = i * RPI + rr;
            const u32x4_t piece = *reinterpret_cast<const u32x4_t*>(stage_rows + r * D + (cc ^ (r & (CPR - 1))) * 8);
            const uint32_t off = (cc * 8 < a.d_qk) ? static_cast<uint32_t>(wr0 + r) * q_stride + cc * 16u : kOutOfRange;
            __builtin_amdgcn_raw_buffer_store_b128(piece, dq_rsrc, static_cast<int>(off), 0, 2);
        }
    }
}

}  // namespace hstu
