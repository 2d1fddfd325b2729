// HSTU jagged attention forward for gfx950 (MI355X): the kernel for small launches of sequences with few query rows -- at
// most 64 -- against keys of any length (a handful of candidates scored against a long history), head-dim slots 64, 128.
//
// With few (sequence, head) items a launch lasts as long as one item, and the other kernels sweep an item's keys one
// 32-key sub-tile after the other in one workgroup whose query tile is mostly empty: batch 16 x 4 heads x 32 rows x 499
// keys takes 14.9 us on the persistent kernel (8 us of start-up, 16 steps).  Here the eight wavefronts of an item's
// workgroup are dealt over its 16-row groups AND over its keys: with one group of rows eight wavefronts take every eighth
// sub-tile each, with two groups four take every fourth, with three or four groups two take every other.  A wavefront
// works alone -- K fragments straight into registers, V sub-tiles into LDS of its own, R blocks in flight, no barrier
// in the sweep -- and the partial outputs of a group's wavefronts are added through LDS at the end, in a fixed order.
//   S^T = K . Q^T (v_mfma_f32_16x16x32), P^T = silu(S^T) masked and rounded, O^T += V^T . P^T: the arithmetic of the
//   kernel for short lists (hstu_fwd_short_kernel.hip.h) step for step; the sum over keys is taken in another order.
// 16-bit inputs, built-in mask (causal with context rows, target rows and target groups) or no mask, no bias.
#pragma once
#include "hstu_bwd_few_rows_kernel.hip.h"
#include "hstu_fwd_short_kernel.hip.h"

namespace hstu {

// K fragments as assembly, like the tile requests of the kernel for short lists and for the same reason: the compiler's
// wait counts across the back edge of the sweep come out as "everything" in front of every fourth block's LDS reads,
// which undoes the prefetch.  The register named here is written when the data arrives; few_rows_wait() is where the
// kernel makes sure of that.
__device__ __forceinline__ void request_fragment(u32x4_t& dst, u32x4_t rsrc, uint32_t voffset)
{
    asm volatile("buffer_load_dwordx4 %0, %1, %2, 0 offen" : "=&v"(dst) : "v"(voffset), "s"(rsrc));
}
// waits until at most OPEN of this wavefront's memory requests are outstanding; the fragments of a block pass through it
// so that nothing that reads them (or LDS: the clobber) moves ahead of the wait
template <int OPEN, int N>
__device__ __forceinline__ void few_rows_wait(u32x4_t (&f)[2][N])
{
    static_assert(OPEN >= 0 && OPEN < 64 && (N == 2 || N == 4), "6 bits of count; head-dim slots 64 and 128");
    if constexpr (N == 2) {
        asm volatile("s_waitcnt vmcnt(%4)" : "+v"(f[0][0]), "+v"(f[0][1]), "+v"(f[1][0]), "+v"(f[1][1]) : "n"(OPEN) : "memory");
    } else {
        asm volatile("s_waitcnt vmcnt(%8)"
                     : "+v"(f[0][0]), "+v"(f[0][1]), "+v"(f[0][2]), "+v"(f[0][3]), "+v"(f[1][0]), "+v"(f[1][1]), "+v"(f[1][2]), "+v"(f[1][3])
                     : "n"(OPEN)
                     : "memory");
    }
}

template <typename Tag, int D>
__global__ __launch_bounds__(kFwdFewRowsThreads, 1) void hstu_fwd_few_rows_kernel(const FwdArgs a)
{
    static_assert(D == 64 || D == 128, "built for the head-dim slots 64 and 128");
    constexpr int WAVES = kFwdFewRowsThreads / 64;
    static_assert(WAVES == 8, "eight wavefronts are dealt over row groups and keys");
    constexpr int R = D == 64 ? 4 : 2;   // blocks in flight per wavefront (registers for K, LDS for V: 128 KiB either way)
    constexpr int SUB_ELEMS = 32 * D;    // one 32-key sub-tile, in 16-bit units
    constexpr int CPR = D / 8;
    constexpr int KSTEPS = D / 32;
    constexpr int MTILES = D / 16;
    constexpr int VLOADS = SUB_ELEMS * 2 / 1024;  // 1 KiB load instructions per V sub-tile (one wavefront loads its own)
    constexpr int kBlockLoads = 2 * KSTEPS + VLOADS;  // memory requests per block and wavefront
    // a block has landed when nothing older than the requests of the R - 1 blocks behind it is open (requests complete in
    // the order of issue; blocks past the last are asked for out of range, so that the count per step is constant)
    constexpr int kOpenBlocks = (R - 1) * kBlockLoads;
    constexpr uint32_t kPastEnd = 0x40000000u;

    // V sub-tiles: stage s of wavefront w at s_v<s> + w * SUB_ELEMS (separate arrays, so that the compiler can tell the
    // stage being filled from the one being read)
    __shared__ __attribute__((aligned(1024))) uint16_t s_v0[WAVES * SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v1[WAVES * SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v2[R == 4 ? WAVES * SUB_ELEMS : 8];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v3[R == 4 ? WAVES * SUB_ELEMS : 8];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = uniform(tid >> 6);
    const int n = lane & 15;
    const int g = lane >> 4;

    uint16_t* const out16 = static_cast<uint16_t*>(a.out);
    const int64_t last_offset = load_index_uniform(a.offs_q, a.n_batch, a.idx64);

    // ---- the item of this workgroup: (sequence, query head) ----
    const int item = static_cast<int>(blockIdx.x);
    const bool in_list = item < a.bh;
    const int b = in_list ? div_small(item, a.n_heads_q) : 0;
    const int h = in_list ? item - b * a.n_heads_q : 0;
    const int hk = div_small(h, a.head_ratio);
    int64_t q0 = 0, q1 = 0, k0 = 0, k1 = 0;
    int n_ctx = 0, n_tgt = 0;
    if (in_list) {
        q0 = load_index_uniform(a.offs_q, b, a.idx64);
        q1 = load_index_uniform(a.offs_q, b + 1, a.idx64);
        k0 = load_index_uniform(a.offs_k, b, a.idx64);
        k1 = load_index_uniform(a.offs_k, b + 1, a.idx64);
        if (a.mask_type == 0) {
            if (a.num_ctx) {
                n_ctx = static_cast<int>(load_index_uniform(a.num_ctx, b, a.idx64));
            }
            if (a.num_tgt) {
                n_tgt = static_cast<int>(load_index_uniform(a.num_tgt, b, a.idx64));
            }
        }
    }
    // defensive clamps: malformed offsets must not turn into out-of-bounds addresses
    q1 = q1 < a.total_q ? q1 : a.total_q;
    k1 = k1 < a.total_k ? k1 : a.total_k;
    q0 = q0 < 0 ? 0 : q0;
    k0 = k0 < 0 ? 0 : k0;
    int sq = static_cast<int>(q1 > q0 ? q1 - q0 : 0);
    int sk = static_cast<int>(k1 > k0 ? k1 - k0 : 0);
    sq = sq < a.max_q ? sq : a.max_q;
    sk = sk < a.max_k ? sk : a.max_k;
    sq = sq < kFewRows ? sq : kFewRows;  // (the host sends no launch with more query rows here)

    if (in_list && sq > 0) {
        if (a.mask_type == 0) {
            n_ctx = n_ctx < 0 ? 0 : n_ctx;
            n_tgt = n_tgt < 0 ? 0 : (n_tgt > sk ? sk : n_tgt);
        }
        const int delta = sk - sq;
        const int hist_k = sk - n_tgt;

        // ---- this wavefront's share: row group `group` (16 rows), every n_splits-th sub-tile from `split` on ----
        const int n_groups = (sq + kShortWaveM - 1) / kShortWaveM;
        const int group_bits = n_groups <= 1 ? 0 : (n_groups == 2 ? 1 : 2);
        const int n_splits = WAVES >> group_bits;
        const int group = wave & ((1 << group_bits) - 1);
        const int split = wave >> group_bits;
        const int wr0 = group * kShortWaveM;
        const bool wave_active = wr0 < sq;

        const uint32_t q_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_qk * 2u;  // bytes per row
        const uint32_t k_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_qk * 2u;
        const uint32_t v_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_v * 2u;
        const uint32_t o_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_v * 2u;
        const __amdgpu_buffer_rsrc_t q_rsrc =
            make_rsrc(static_cast<const uint8_t*>(a.q) + (q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_qk) * 2,
                      static_cast<uint32_t>(sq - 1) * q_stride + a.d_qk * 2u);
        const u32x4_t k_rsrc =
            make_rsrc_words(static_cast<const uint8_t*>(a.k) + (k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_qk) * 2,
                            sk > 0 ? static_cast<uint32_t>(sk - 1) * k_stride + a.d_qk * 2u : 0u);
        const u32x4_t v_rsrc =
            make_rsrc_words(static_cast<const uint8_t*>(a.v) + (k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_v) * 2,
                            sk > 0 ? static_cast<uint32_t>(sk - 1) * v_stride + a.d_v * 2u : 0u);
        const __amdgpu_buffer_rsrc_t o_rsrc = make_rsrc(out16 + (q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_v),
                                                        static_cast<uint32_t>(sq - 1) * o_stride + a.d_v * 2u);

        // Q fragment (B operand of the first product): lane (n, g) holds Q[row n][32 js + 8 g .. + 7]
        u32x4_t qf[KSTEPS];
        {
            const uint32_t row_off = static_cast<uint32_t>(wr0 + n) * q_stride;
#pragma unroll
            for (int js = 0; js < KSTEPS; ++js) {
                const int d0 = 32 * js + 8 * g;
                const uint32_t off = (d0 < a.d_qk) ? row_off + d0 * 2u : kOutOfRange;
                qf[js] = __builtin_amdgcn_raw_buffer_load_b128(q_rsrc, static_cast<int>(off), 0, 0);
            }
        }

        // ---- per-row visibility: visible(j) = j < lim && !(hole_lo <= j < hole_hi); the wavefront's last visible key ----
        int row = wr0 + n;
        row = row < sq - 1 ? row : sq - 1;
        int lim;
        int hole_lo = 0;
        int hole_hi = 0;
        int lim_wave;  // no row of this wavefront sees a key from here on
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
            const int last_row = (wr0 + kShortWaveM < sq ? wr0 + kShortWaveM : sq) - 1;
            lim_wave = last_row + delta + 1;
            if (wr0 < n_ctx) {
                lim_wave = lim_wave > hist_k ? lim_wave : hist_k;
            }
            lim_wave = lim_wave < 0 ? 0 : (lim_wave > sk ? sk : lim_wave);
        } else {
            lim = sk;
            lim_wave = sk;
        }
        const int nx_w = wave_active ? (lim_wave + 31) / 32 : 0;
        // bounds relative to the lane's first key (key = c0 + 16 j + 4 g + r)
        const int lim_lane = lim - 4 * g;
        const int hole_lo_lane = hole_lo - 4 * g;
        const int hole_hi_lane = hole_hi - 4 * g;

        // ---- loads of a block: K fragments (A operand: lane (n, g) holds K[key 16 j + n][32 js + 8 g .. + 7]) into the
        // registers of slot S, the V sub-tile into this wavefront's part of stage S; piece 64 i + lane of a sub-tile is row
        // piece / CPR, physical chunk piece % CPR, which holds the logical chunk the swizzle names.  Keys past the sequence
        // and dims past the head dim read as zeros; blocks past the wavefront's last are sent out of range ----
        u32x4_t kr[R][2][KSTEPS];
        auto v_stage = [&](auto ic) -> uint16_t* {
            constexpr int S = decltype(ic)::value;
            uint16_t* const base = S == 0 ? s_v0 : (S == 1 ? s_v1 : (S == 2 ? s_v2 : s_v3));
            return base + wave * SUB_ELEMS;
        };
        uint32_t v_src[VLOADS];
#pragma unroll
        for (int i = 0; i < VLOADS; ++i) {
            const int piece = i * 64 + lane;
            const int r = piece / CPR;
            const int vc = few_rows_swizzle<D>(r, piece % CPR);
            v_src[i] = (vc * 8 < a.d_v) ? static_cast<uint32_t>(r) * v_stride + vc * 16u : kOutOfRange;
        }
        auto load_block = [&](auto ic, int x) {
            constexpr int S = decltype(ic)::value;
            const uint32_t past = x < nx_w ? 0u : kPastEnd;
            const uint32_t kb = static_cast<uint32_t>(x * 32 + n) * k_stride + past;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
#pragma unroll
                for (int js = 0; js < KSTEPS; ++js) {
                    const int d0 = 32 * js + 8 * g;
                    const uint32_t off = (d0 < a.d_qk) ? kb + static_cast<uint32_t>(16 * j) * k_stride + d0 * 2u : kOutOfRange;
                    request_fragment(kr[S][j][js], k_rsrc, off);
                }
            }
            const uint32_t vb = static_cast<uint32_t>(x * 32) * v_stride + past;
            const uint32_t dst = lds_address(v_stage(ic));
#pragma unroll
            for (int i = 0; i < VLOADS; ++i) {
                request_to_lds_b128(v_rsrc, dst + i * 1024u, v_src[i] + vb);
            }
        };

        f32x4_t o_acc[MTILES];
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
            o_acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
        const float c_exp = a.c_exp;
        const int vr = 4 * g + (n >> 2);
        const int v_row_off = vr * D + 4 * (n & 1);
        const int v_chunk_lo = (n & 3) >> 1;

        auto step = [&](auto ic, int x) {
            constexpr int S = decltype(ic)::value;
            const int c0 = x * 32;
            // the block has landed: fragments in their registers, V rows in this wavefront's part of the stage
            few_rows_wait<kOpenBlocks>(kr[S]);
            // S^T (32 keys x 16 rows) = K . Q^T: two blocks of 16 keys
            f32x4_t s0 = {0.f, 0.f, 0.f, 0.f};
            f32x4_t s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int js = 0; js < KSTEPS; ++js) {
                s0 = mfma16<Tag>(kr[S][0][js], qf[js], s0);
                s1 = mfma16<Tag>(kr[S][1][js], qf[js], s1);
            }
            // P^T = silu(S^T), masked, rounded: element (j, r) is key c0 + 16 j + 4 g + r of this lane's row
            float p[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float s = e < 4 ? s0[e] : s1[e - 4];
                float tt = __builtin_amdgcn_exp2f(s * c_exp);
                tt = __builtin_amdgcn_rcpf(1.0f + tt);
                const int kk = c0 + 16 * (e / 4) + (e % 4);  // + 4 g is folded into the *_lane bounds
                const bool vis = (kk < lim_lane) && !(kk >= hole_lo_lane && kk < hole_hi_lane);
                p[e] = vis ? s * tt : 0.f;
            }
            const u32x4_t pb = {pack2<Tag>(p[0], p[1]), pack2<Tag>(p[2], p[3]), pack2<Tag>(p[4], p[5]), pack2<Tag>(p[6], p[7])};
            // O^T (D dims x 16 rows) += V^T . P^T
            const uint16_t* const vt = v_stage(ic);
#pragma unroll
            for (int mt = 0; mt < MTILES; ++mt) {
                const uint16_t* const vp = vt + v_row_off + few_rows_swizzle<D>(vr, 2 * mt + v_chunk_lo) * 8;
                const u32x2_t lo = lds_read_tr16_b64(vp);
                const u32x2_t hi = lds_read_tr16_b64(vp + 16 * D);
                const u32x4_t va = {lo[0], lo[1], hi[0], hi[1]};
                o_acc[mt] = mfma16<Tag>(va, pb, o_acc[mt]);
            }
            // the slot is free (its LDS reads fed the products above): the block R rounds on
            __builtin_amdgcn_sched_barrier(0);
            load_block(ic, x + R * n_splits);
        };

        typedef std::integral_constant<int, 0> ic0_t;
        typedef std::integral_constant<int, 1> ic1_t;
        typedef std::integral_constant<int, 2> ic2_t;
        typedef std::integral_constant<int, 3> ic3_t;
        {
            int x = split;
            load_block(ic0_t{}, x);
            load_block(ic1_t{}, x + n_splits);
            if constexpr (R == 4) {
                load_block(ic2_t{}, x + 2 * n_splits);
                load_block(ic3_t{}, x + 3 * n_splits);
            }
            // (the compiler counts the Q loads but not these requests: everything is in before the sweep)
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt((0 & 15) | (7 << 4) | (15 << 8));
            __builtin_amdgcn_sched_barrier(0);
            while (x < nx_w) {
                step(ic0_t{}, x);
                x += n_splits;
                if (x >= nx_w) {
                    break;
                }
                step(ic1_t{}, x);
                x += n_splits;
                if constexpr (R == 4) {
                    if (x >= nx_w) {
                        break;
                    }
                    step(ic2_t{}, x);
                    x += n_splits;
                    if (x >= nx_w) {
                        break;
                    }
                    step(ic3_t{}, x);
                    x += n_splits;
                }
            }
        }

        // ---- the partial outputs of a row group's wavefronts, added in the order of the splits: each leaves its own in
        // its part of stage 0.  Every request has landed by then -- the last ones were sent out of range and write zeros,
        // into LDS and into the fragment registers, which stay the fragments' until here ----
        few_rows_wait<0>(kr[0]);
        few_rows_wait<0>(kr[1]);
        if constexpr (R == 4) {
            few_rows_wait<0>(kr[2]);
            few_rows_wait<0>(kr[3]);
        }
        float* const mine = reinterpret_cast<float*>(s_v0 + wave * SUB_ELEMS);
        static_assert(SUB_ELEMS * 2 >= MTILES * 64 * 16, "a wavefront's partial output fits its part of a stage");
        if (split != 0) {
#pragma unroll
            for (int mt = 0; mt < MTILES; ++mt) {
                *reinterpret_cast<f32x4_t*>(mine + (mt * 64 + lane) * 4) = o_acc[mt];
            }
        }
        __syncthreads();
        if (split == 0 && wave_active) {
            for (int s = 1; s < n_splits; ++s) {
                const float* const other = reinterpret_cast<const float*>(s_v0 + ((s << group_bits) + group) * SUB_ELEMS);
#pragma unroll
                for (int mt = 0; mt < MTILES; ++mt) {
                    const f32x4_t t = *reinterpret_cast<const f32x4_t*>(other + (mt * 64 + lane) * 4);
                    o_acc[mt] += t;
                }
            }
            // ---- store O: lane (n, g) holds dims 16 mt + 4 g + 0..3 of query row wr0 + n ----
            const float c_out = a.c_out;
            if (a.out_vec_ok != 0) {
                uint16_t* const stage = s_v1 + wave * SUB_ELEMS;  // (this wavefront's own)
#pragma unroll
                for (int mt = 0; mt < MTILES; ++mt) {
                    u32x2_t w;
                    w[0] = pack2<Tag>(o_acc[mt][0] * c_out, o_acc[mt][1] * c_out);
                    w[1] = pack2<Tag>(o_acc[mt][2] * c_out, o_acc[mt][3] * c_out);
                    const int chunk = (2 * mt + (g >> 1)) ^ (n & (CPR - 1));
                    *reinterpret_cast<u32x2_t*>(stage + n * D + chunk * 8 + 4 * (g & 1)) = w;
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                constexpr int RPI = 64 / CPR;  // rows per store instruction
                const int rr = lane / CPR;
                const int cc = lane % CPR;
#pragma unroll
                for (int i = 0; i < kShortWaveM / RPI; ++i) {
                    const int r = i * RPI + rr;
                    const u32x4_t piece = *reinterpret_cast<const u32x4_t*>(stage + r * D + (cc ^ (r & (CPR - 1))) * 8);
                    const uint32_t off = (cc * 8 < a.d_v) ? static_cast<uint32_t>(wr0 + r) * o_stride + cc * 16u : kOutOfRange;
                    __builtin_amdgcn_raw_buffer_store_b128(piece, o_rsrc, static_cast<int>(off), 0, 0);
                }
            } else {
                const uint32_t row_off = static_cast<uint32_t>(wr0 + n) * o_stride;
#pragma unroll
                for (int mt = 0; mt < MTILES; ++mt) {
                    const int d0 = 16 * mt + 4 * g;
                    const uint32_t off = (d0 < a.d_v) ? row_off + d0 * 2u : kOutOfRange;
                    u32x2_t w;
                    w[0] = pack2<Tag>(o_acc[mt][0] * c_out, o_acc[mt][1] * c_out);
                    w[1] = pack2<Tag>(o_acc[mt][2] * c_out, o_acc[mt][3] * c_out);
                    __builtin_amdgcn_raw_buffer_store_b64(w, o_rsrc, static_cast<int>(off), 0, 0);
                }
            }
        }
    }

    // ---- rows past the last offset belong to no sequence: zero-fill (all workgroups share the job) ----
    {
        const int64_t first_tail = last_offset < 0 ? 0 : (last_offset < a.total_q ? last_offset : a.total_q);
        const int64_t row_elems = static_cast<int64_t>(a.n_heads_q) * a.d_v;
        const int64_t n_tail = (a.total_q - first_tail) * row_elems;
        uint16_t* tail = out16 + first_tail * row_elems;
        for (int64_t e = static_cast<int64_t>(blockIdx.x) * kFwdFewRowsThreads + tid; e < n_tail;
             e += static_cast<int64_t>(gridDim.x) * kFwdFewRowsThreads) {
            tail[e] = 0;
        }
    }
}

}  // namespace hstu
