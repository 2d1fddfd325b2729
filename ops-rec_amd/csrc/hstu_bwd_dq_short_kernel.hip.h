// HSTU jagged attention backward for gfx950 (MI355X): the query-tile kernel (dQ; dS and P for the key-tile
// workgroups that read them back) for short rows.
//
// hstu_bwd_dq_kernel gives a wavefront 32 query rows; one of its steps over a 32-key sub-tile -- S^T = K Q^T,
// dP^T = V dO^T, dS, dQ^T += K^T dS^T: 48 matrix instructions and the score algebra of 1024 elements -- takes about
// 1.5 us whatever else runs on the CU, and a launch lasts as long as its longest row of steps (keys / 32 of them): at
// batch 32 x 4 heads, lengths 256..1024, 68 us for work that would fill the machine for 25.  This kernel is the same
// computation with 16 query rows per wavefront (v_mfma_f32_16x16x32): a step is half the work and half as long, three
// wavefronts share a SIMD, and a workgroup of four wavefronts takes a 64-row query tile, so the grid has twice as
// many, shorter items.  One workgroup per (64-row tile, sequence, head) slot, heaviest tiles first, all tiles of a
// (sequence, K/V head) pair on one XCD (see the forward kernel for short lists, whose scheme this is).
//
// It pays 1.5 times the matrix-pipe time per product term and twice the LDS operand traffic, so it is the faster one
// only while rows are short; 16-bit inputs, head-dim slot 128, no bias, no custom mask.
//
// STORE 0: dQ only.  STORE 1: dS also goes to a workspace in the layout of the attn_bias gradient ([max_q][max_k] per
// sequence and head), for dK workgroups that read it back.  STORE 2: dS and P also go to the plane the key-tile workgroups of the next launch read (layout of
// hstu_bwd_dq_kernel: per query row and 32-key block, 32 dS values then 32 P values, one 128-byte line).  A block is
// written for a row whenever the 32-row group of the row can see it -- the unit by which the readers decide what to
// read -- with zeros where this wavefront's own 16 rows cannot.
//
// Formula: ascendc/attention/hstu_v1/hstu_backward_v1/op_kernel/vector_score.h:159-205.
#pragma once
#include "hstu_bwd_kernel.hip.h"
#include "hstu_fwd_short_kernel.hip.h"

namespace hstu {

constexpr int kDqShortWavesPerSimd = 3;

// K sub-tile in LDS, read plainly (A operand of S^T: 16 consecutive rows, one 16-byte chunk each) and transposed (A
// operand of dQ^T: rows 4 g .. 4 g + 3 of two neighbouring groups, 32 bytes each): the XOR term is a bijection of the
// low four row bits (the plain read hits 16 different chunks) whose upper three bits tell rows 0..7 apart (the eight
// 32-byte pieces of a transposed read fall into different bank groups).  Adding 16 to the row leaves it alone.  (Rows of
// 256 elements: the same term over each half of the row's 32 chunks.)
template <int D>
__device__ __forceinline__ int both_ways16_swizzle(int row, int chunk)
{
    static_assert(D == 128 || D == 256, "16 or 32 chunks of 16 bytes per row");
    return chunk ^ (((row & 7) << 1) | ((row >> 3) & 1));
}

template <typename Tag, int D, int STORE>
__global__ __launch_bounds__(kDqShortThreads, kDqShortWavesPerSimd) void hstu_bwd_dq_short_kernel(const BwdArgs a)
{
    static_assert(D == 128, "built for the head-dim slot 128");
    static_assert(STORE >= 0 && STORE <= 2, "dQ only; with dS in the bias layout; with the dS / P plane");
    constexpr bool WANT_P = STORE == 2;
    constexpr bool WANT_DS = STORE == 1;
    constexpr int SUB_ELEMS = 32 * D;
    constexpr int CPR = D / 8;
    constexpr int KSTEPS = D / 32;
    constexpr int MTILES = D / 16;
    constexpr int LPW = 32 * D * 2 / 1024 / 4;  // 1 KiB load instructions per wavefront and sub-tile (K, and again V)
    static_assert(LPW == 2, "two load instructions per wavefront for K and two for V");
    constexpr int kWaitStage = ((2 * LPW) & 15) | (7 << 4) | (15 << 8);  // the requests of one later step may be open
    constexpr uint32_t kPastEnd = 0x40000000u;

    // three stages of {K, V} sub-tiles (sub-tile x in stage x mod 3)
    __shared__ __attribute__((aligned(1024))) uint16_t s_k0[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_k1[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_k2[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v0[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v1[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v2[SUB_ELEMS];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = uniform(tid >> 6);
    const int n = lane & 15;
    const int g = lane >> 4;

    zero_tail_rows(a.dq, a.offs_q, a.n_batch, a.idx64, a.total_q, static_cast<int64_t>(a.n_heads_q) * a.d_qk, kDqShortThreads);

    // (the levels that exist in the batch, at most those the host sized the grid for: see batch_max_rows)
    const int n_levels = live_levels(a, lane, kDqShortRows, (a.max_q + kDqShortRows - 1) / kDqShortRows);
    const int n_pairs = a.n_batch * a.n_heads_k;
    const ShortSlot slot = short_slot(static_cast<int>(blockIdx.x), n_pairs, a.head_ratio);
    if (slot.pair >= n_pairs || slot.level >= n_levels) {
        return;
    }
    const int b = div_small(slot.pair, a.n_heads_k);
    const int hk = slot.pair - b * a.n_heads_k;
    const int h = hk * a.head_ratio + slot.r;
    // (heaviest tiles first; with context rows the first tile of a sequence sweeps all of its history keys and goes ahead)
    const int qt = (a.mask_type == 0 && a.num_ctx != nullptr) ? (slot.level == 0 ? 0 : n_levels - slot.level) : n_levels - 1 - slot.level;
    const SeqInfo sq_info = load_seq(a, b);
    const int sq = sq_info.sq, sk = sq_info.sk;
    const int r0 = qt * kDqShortRows;
    if (r0 >= sq) {
        return;
    }
    const int wr0 = r0 + wave * kShortWaveM;

    const uint32_t q_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_qk * 2u;
    const uint32_t g_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_v * 2u;
    const uint32_t k_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_qk * 2u;
    const uint32_t v_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_v * 2u;
    const __amdgpu_buffer_rsrc_t q_rsrc =
        make_rsrc(static_cast<const uint8_t*>(a.q) + (sq_info.q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_qk) * 2,
                  static_cast<uint32_t>(sq - 1) * q_stride + a.d_qk * 2u);
    const __amdgpu_buffer_rsrc_t g_rsrc =
        make_rsrc(static_cast<const uint8_t*>(a.grad) + (sq_info.q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_v) * 2,
                  static_cast<uint32_t>(sq - 1) * g_stride + a.d_v * 2u);
    const __amdgpu_buffer_rsrc_t dq_rsrc =
        make_rsrc(static_cast<uint8_t*>(a.dq) + (sq_info.q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_qk) * 2,
                  static_cast<uint32_t>(sq - 1) * q_stride + a.d_qk * 2u);
    const u32x4_t k_rsrc =
        make_rsrc_words(static_cast<const uint8_t*>(a.k) + (sq_info.k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_qk) * 2,
                        sk > 0 ? static_cast<uint32_t>(sk - 1) * k_stride + a.d_qk * 2u : 0u);
    const u32x4_t v_rsrc =
        make_rsrc_words(static_cast<const uint8_t*>(a.v) + (sq_info.k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_v) * 2,
                        sk > 0 ? static_cast<uint32_t>(sk - 1) * v_stride + a.d_v * 2u : 0u);

    // per-lane source offsets of the sub-tile loads: 16-byte piece -> row, swizzled chunk (the swizzle is its own inverse)
    uint32_t k_src[LPW], v_src[LPW];
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
        const int piece = (wave * LPW + i) * 64 + lane;
        const int r = piece / CPR;
        const int pc = piece % CPR;
        const int cs = both_ways16_swizzle<D>(r, pc);
        k_src[i] = (cs * 8 < a.d_qk) ? static_cast<uint32_t>(r) * k_stride + cs * 16u : kOutOfRange;
        v_src[i] = (cs * 8 < a.d_v) ? static_cast<uint32_t>(r) * v_stride + cs * 16u : kOutOfRange;
    }
    // LDS read offsets relative to a sub-tile, in elements: plain read of row n (+ 16), MFMA step js; transposed read of
    // rows 4 g .. 4 g + 3 (+ 16), dims 16 mt .. + 15
    int n_lane_off[KSTEPS];
#pragma unroll
    for (int js = 0; js < KSTEPS; ++js) {
        n_lane_off[js] = n * D + both_ways16_swizzle<D>(n, 4 * js + g) * 8;
    }
    const int vr = 4 * g + (n >> 2);
    const int t_row_off = vr * D + 4 * (n & 1);
    const int t_chunk_lo = (n & 3) >> 1;
    auto t_lane_off = [&](int mt) -> int { return t_row_off + both_ways16_swizzle<D>(vr, 2 * mt + t_chunk_lo) * 8; };

    // keys needed by this tile
    int kmax;
    if (a.mask_type == 0) {
        const int r1 = (r0 + kDqShortRows < sq) ? r0 + kDqShortRows : sq;
        kmax = r1 + sq_info.delta;
        if (r0 < sq_info.n_ctx) {
            kmax = kmax > sq_info.hist_k ? kmax : sq_info.hist_k;
        }
        kmax = kmax < 0 ? 0 : (kmax > sk ? sk : kmax);
    } else {
        kmax = sk;
    }
    const int n_sub = (kmax + 31) / 32;

    auto k_stage = [&](int i) -> uint16_t* { return i == 0 ? s_k0 : (i == 1 ? s_k1 : s_k2); };
    auto v_stage = [&](int i) -> uint16_t* { return i == 0 ? s_v0 : (i == 1 ? s_v1 : s_v2); };
    auto request = [&](uint16_t* kd, uint16_t* vd, int x) {
        const uint32_t past = x < n_sub ? 0u : kPastEnd;
        const uint32_t kb = static_cast<uint32_t>(x * 32) * k_stride + past;
        const uint32_t vb = static_cast<uint32_t>(x * 32) * v_stride + past;
#pragma unroll
        for (int i = 0; i < LPW; ++i) {
            request_to_lds_b128(k_rsrc, lds_address(kd) + (wave * LPW + i) * 1024u, k_src[i] + kb);
            request_to_lds_b128(v_rsrc, lds_address(vd) + (wave * LPW + i) * 1024u, v_src[i] + vb);
        }
    };

    // ---- start-up: the first sub-tile, the resident rows (Q and dO fragments, B operands), the second sub-tile ----
    request(s_k0, s_v0, 0);
    u32x4_t qf[KSTEPS], gf[KSTEPS];
    {
        const uint32_t q_off = static_cast<uint32_t>(wr0 + n) * q_stride;
        const uint32_t g_off = static_cast<uint32_t>(wr0 + n) * g_stride;
#pragma unroll
        for (int js = 0; js < KSTEPS; ++js) {
            const int d0 = 32 * js + 8 * g;
            qf[js] = __builtin_amdgcn_raw_buffer_load_b128(q_rsrc, static_cast<int>(d0 < a.d_qk ? q_off + d0 * 2u : kOutOfRange), 0, 0);
            gf[js] = __builtin_amdgcn_raw_buffer_load_b128(g_rsrc, static_cast<int>(d0 < a.d_v ? g_off + d0 * 2u : kOutOfRange), 0, 0);
        }
    }
    request(s_k1, s_v1, 1);

    int row = wr0 + n;
    row = row < sq - 1 ? row : sq - 1;
    int lim, hole_lo, hole_hi;
    row_bounds(sq_info, a.mask_type, a.target_group, row, lim, hole_lo, hole_hi);
    const WaveBounds wb =
        wave_bounds(a.mask_type, wr0, sq, sk, sq_info.n_ctx, sq_info.n_tgt, a.target_group, wr0 < sq, kShortWaveM);
    const int nx_w = (wb.lim_max + 31) / 32;
    // the blocks the 32-row group of this wavefront's rows can see: what the readers of the plane take as written
    const int nx_store = (swept_key_limit(a, sq_info, wr0 & ~31) + 31) / 32;
    const int lim_lane = lim - 4 * g;
    const int hole_lo_lane = hole_lo - 4 * g;
    const int hole_hi_lane = hole_hi - 4 * g;

    const __amdgpu_buffer_rsrc_t p_rsrc =
        make_rsrc(WANT_P ? pair_plane_of(a, sq_info.q0, b, h) : nullptr, WANT_P ? pair_seq_bytes(a, sq) : 0u);
    const uint32_t pair_row_off = (WANT_P && wr0 + n < sq) ? pair_row_offset(a, wr0 + n) : kOutOfRange;

    // STORE 1: dS in the bias layout
    const uint32_t bias_bytes = static_cast<uint32_t>(a.max_q) * static_cast<uint32_t>(a.max_k) * 2u;
    const __amdgpu_buffer_rsrc_t ds_rsrc =
        make_rsrc(WANT_DS ? static_cast<uint16_t*>(a.drab) + (static_cast<int64_t>(b) * a.n_heads_q + h) * a.max_q * static_cast<int64_t>(a.max_k)
                          : nullptr,
                  WANT_DS ? bias_bytes : 0u);
    const uint32_t bias_row_off = (wr0 + n < sq) ? static_cast<uint32_t>(wr0 + n) * static_cast<uint32_t>(a.max_k) * 2u : kOutOfRange;
    auto store_ds = [&](int x, uint32_t ds0, uint32_t ds1, uint32_t ds2, uint32_t ds3) {
        const int c0 = x * 32;
        const uint32_t base = bias_row_off + static_cast<uint32_t>(c0 + 4 * g) * 2u;
        const bool in0 = c0 + 8 * (g >> 1) < sk;
        const bool in1 = c0 + 16 + 8 * (g >> 1) < sk;
        const u32x2_t a0 = {ds0, ds1}, a1 = {ds2, ds3};
        __builtin_amdgcn_raw_buffer_store_b64(a0, ds_rsrc, static_cast<int>(in0 ? base : kOutOfRange), 0, 0);
        __builtin_amdgcn_raw_buffer_store_b64(a1, ds_rsrc, static_cast<int>(in1 ? base + 32u : kOutOfRange), 0, 0);
    };

    f32x4_t dq_acc[MTILES];
#pragma unroll
    for (int mt = 0; mt < MTILES; ++mt) {
        dq_acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    const ScoreConsts sconst = score_consts(a.alpha, a.scale);

    // the four 8-byte pieces of this lane in the 128-byte line of (row, block x): dS of keys 4 g .. + 3 and 16 + 4 g .. + 3,
    // then P of the same keys.  A piece goes out when the 8-key group it lies in starts inside the sequence (the unit
    // by which the readers predicate their 16-byte reads).
    auto store_line = [&](int x, uint32_t ds0, uint32_t ds1, uint32_t ds2, uint32_t ds3, uint32_t p0, uint32_t p1, uint32_t p2,
                          uint32_t p3) {
        const int c0 = x * 32;
        const uint32_t base = pair_row_off + static_cast<uint32_t>(2 * c0 + 4 * g) * 2u;
        const bool in0 = c0 + 8 * (g >> 1) < sk;
        const bool in1 = c0 + 16 + 8 * (g >> 1) < sk;
        const u32x2_t a0 = {ds0, ds1}, a1 = {ds2, ds3}, b0 = {p0, p1}, b1 = {p2, p3};
        __builtin_amdgcn_raw_buffer_store_b64(a0, p_rsrc, static_cast<int>(in0 ? base : kOutOfRange), 0, 0);
        __builtin_amdgcn_raw_buffer_store_b64(a1, p_rsrc, static_cast<int>(in1 ? base + 32u : kOutOfRange), 0, 0);
        __builtin_amdgcn_raw_buffer_store_b64(b0, p_rsrc, static_cast<int>(in0 ? base + 64u : kOutOfRange), 0, 0);
        __builtin_amdgcn_raw_buffer_store_b64(b1, p_rsrc, static_cast<int>(in1 ? base + 96u : kOutOfRange), 0, 0);
    };

    auto step = [&](const uint16_t* kn, const uint16_t* vn, uint16_t* kn_o, uint16_t* vn_o, int x) {
        // sub-tile x has landed (mine, then everybody's), and nobody reads the stage of step x - 1 any more
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(kWaitStage);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        request(kn_o, vn_o, x + 2);
        if (x >= nx_w) {
            if (x < nx_store) {  // visible to the other half of the 32-row group only
                if constexpr (WANT_P) {
                    store_line(x, 0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u);
                }
                if constexpr (WANT_DS) {
                    store_ds(x, 0u, 0u, 0u, 0u);
                }
            }
            return;
        }
        const int c0 = x * 32;
        // S^T = K Q^T and dP^T = V dO^T (32 keys x 16 rows each, two blocks of 16 keys)
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
        // dS (and P): element (j, r) is key c0 + 16 j + 4 g + r of this lane's row
        float ds[8], pv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float sv = e < 4 ? s0[e] : s1[e - 4];
            const float dv = e < 4 ? dp0[e] : dp1[e - 4];
            ds[e] = score_ds(sv, dv, sconst);
            pv[e] = WANT_P ? score_p(sv, sconst) : 0.f;
        }
        const bool full = (c0 + 32 <= wb.lim_min) && !(wb.any_hole && c0 + 32 > sq_info.hist_k && c0 < wb.hole_hi_max);
        if (!full) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int kk = c0 + 16 * (e / 4) + (e % 4);  // + 4 g is folded into the *_lane bounds
                const bool vis = (kk < lim_lane) && !(kk >= hole_lo_lane && kk < hole_hi_lane);
                ds[e] = vis ? ds[e] : 0.f;
                pv[e] = vis ? pv[e] : 0.f;
            }
        }
        const u32x4_t db = {pack2<Tag>(ds[0], ds[1]), pack2<Tag>(ds[2], ds[3]), pack2<Tag>(ds[4], ds[5]),
                            pack2<Tag>(ds[6], ds[7])};
        if constexpr (WANT_P) {
            store_line(x, db[0], db[1], db[2], db[3], pack2<Tag>(pv[0], pv[1]), pack2<Tag>(pv[2], pv[3]),
                       pack2<Tag>(pv[4], pv[5]), pack2<Tag>(pv[6], pv[7]));
        }
        if constexpr (WANT_DS) {
            store_ds(x, db[0], db[1], db[2], db[3]);
        }
        // dQ^T (D dims x 16 rows) += K^T dS^T
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
            const uint16_t* const kp = kn + t_lane_off(mt);
            const u32x2_t lo = lds_read_tr16_b64(kp);
            const u32x2_t hi = lds_read_tr16_b64(kp + 16 * D);
            const u32x4_t ka = {lo[0], lo[1], hi[0], hi[1]};
            dq_acc[mt] = mfma16<Tag>(ka, db, dq_acc[mt]);
        }
    };

    // Everything asked for so far is in before the first step (the count must be zero here: the compiler counts the
    // Q / dO loads but not the tile requests, see the forward kernel for short lists); the first step's own wait is
    // then trivially met.
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt((0 & 15) | (7 << 4) | (15 << 8));
    __builtin_amdgcn_sched_barrier(0);
    if (n_sub > 0) {
        int x = 0;
        while (true) {  // (step x reads stage x mod 3 and has stage (x + 2) mod 3 filled)
            step(s_k0, s_v0, s_k2, s_v2, x);
            if (++x >= n_sub) {
                break;
            }
            step(s_k1, s_v1, s_k0, s_v0, x);
            if (++x >= n_sub) {
                break;
            }
            step(s_k2, s_v2, s_k1, s_v1, x);
            if (++x >= n_sub) {
                break;
            }
        }
    }

    // ---- store dQ: lane (n, g) holds dims 16 mt + 4 g + 0..3 of query row wr0 + n ----
    if (a.grad_vec_ok != 0) {
        // (every wavefront is done with the ring, and every request has landed, before anybody writes into a stage)
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        uint16_t* const stage = k_stage(wave < 3 ? wave : 0) + (wave == 3 ? 16 * D : 0);  // 4 KiB per wavefront
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
        constexpr int kNonTemporal = 2;
        const int rr = lane / CPR;
        const int cc = lane % CPR;
#pragma unroll
        for (int i = 0; i < kShortWaveM / RPI; ++i) {
            const int r = i * RPI + rr;
            const u32x4_t piece = *reinterpret_cast<const u32x4_t*>(stage + r * D + (cc ^ r) * 8);
            const uint32_t off = (cc * 8 < a.d_qk) ? static_cast<uint32_t>(wr0 + r) * q_stride + cc * 16u : kOutOfRange;
            __builtin_amdgcn_raw_buffer_store_b128(piece, dq_rsrc, static_cast<int>(off), 0, kNonTemporal);
        }
    } else {
        const uint32_t row_off = static_cast<uint32_t>(wr0 + n) * q_stride;
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
            const int d0 = 16 * mt + 4 * g;
            const uint32_t off = (d0 < a.d_qk) ? row_off + d0 * 2u : kOutOfRange;
            u32x2_t w;
            w[0] = pack2<Tag>(dq_acc[mt][0], dq_acc[mt][1]);
            w[1] = pack2<Tag>(dq_acc[mt][2], dq_acc[mt][3]);
            __builtin_amdgcn_raw_buffer_store_b64(w, dq_rsrc, static_cast<int>(off), 0, 0);
        }
    }
}

}  // namespace hstu
