// HSTU jagged attention forward for gfx950 (MI355X): the kernel for batches of tiny sequences -- no sequence longer
// than ROWS = 32 or 64 rows or keys (max_seq_len_q, max_seq_len_k <= ROWS), head-dim slots 64, 128 and 256.
//
// Such a launch is bound by memory and by latency, not by the products: a (sequence, head) item reads 3 x 32 rows and
// writes 32, and its two products are one 32-key sub-tile.  The persistent kernel spends a whole 128-row workgroup and
// about 8 us of start-up on each item, one after the other (batch 2048, 2 heads, head dim 256, 32 rows: 135 us for
// 268 MB of operands; batch 2048, 4 heads, head dim 64, 48 rows: 118 us for 201 MB).  Here an item is a workgroup of
// ROWS / 16 wavefronts of 16 query rows each with 2 x ROWS x D x 2 bytes of LDS (32 KiB at 32 rows and head dim 256), so
// several workgroups share a CU and overlap each other's load, product and store phases; nothing is pipelined inside an item:
//   K and V rows (zeros past the sequence) -> LDS by direct-to-LDS loads, Q fragment -> registers, one wait, one barrier;
//   S^T = K . Q^T (v_mfma_f32_16x16x32), P^T = silu(S^T) masked and rounded, O^T = V^T . P^T (V^T by transposing LDS
//   reads), the arithmetic of the kernel for short lists (hstu_fwd_short_kernel.hip.h) step for step;
//   output rows through LDS, whole 128-byte lines per store instruction.
// 16-bit inputs, built-in mask (causal with context rows, target rows and target groups) or no mask, no bias.
#pragma once
#include "hstu_bwd_few_rows_kernel.hip.h"
#include "hstu_fwd_short_kernel.hip.h"

namespace hstu {

// wavefronts per SIMD the variants are compiled for (LDS: 4 ROWS D bytes per workgroup of ROWS / 16 wavefronts)
constexpr int tiny_waves_per_simd(int d, int rows) { return rows == 32 ? (d <= 128 ? 4 : 3) : (d <= 128 ? 4 : 2); }

// one LDS layout for the plain reads of K rows and the transposing reads of V rows, by head-dim slot
template <int D>
__device__ __forceinline__ int tiny_swizzle(int row, int chunk)
{
    if constexpr (D == 64) {
        return both_ways16_swizzle64(row, chunk);
    } else {
        return both_ways16_swizzle<D>(row, chunk);
    }
}

template <typename Tag, int D, int ROWS>
__global__ __launch_bounds__(ROWS * 4, tiny_waves_per_simd(D, ROWS)) void hstu_fwd_tiny_kernel(const FwdArgs a)
{
    static_assert(D == 64 || D == 128 || D == 256, "built for the head-dim slots 64, 128 and 256");
    static_assert(ROWS == 32 || ROWS == 64, "sequences of at most 32 or 64 rows and keys");
    constexpr int WAVES = ROWS / kShortWaveM;
    constexpr int THREADS = WAVES * 64;
    constexpr int TILE_ELEMS = ROWS * D;  // all keys of an item, in 16-bit units
    constexpr int CPR = D / 8;            // 16-byte chunks per row
    constexpr int KSTEPS = D / 32;        // MFMA steps over the head dim (QK product)
    constexpr int MTILES = D / 16;        // 16-wide output tiles over the head dim (PV product)
    constexpr int LOADS = TILE_ELEMS * 2 / 1024 / WAVES;  // 1 KiB load instructions per wavefront and tile

    __shared__ __attribute__((aligned(1024))) uint16_t s_k[TILE_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v[TILE_ELEMS];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = uniform(tid >> 6);
    const int n = lane & 15;  // query row of the wavefront / key row of a 16-key block / output dim of a tile
    const int g = lane >> 4;  // which 8 of the 32 contraction values, which 4 of the 16 accumulator rows

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
    sq = sq < ROWS ? sq : ROWS;  // (the host sends no launch with longer sequences here)
    sk = sk < ROWS ? sk : ROWS;

    if (in_list && sq > 0) {
        if (a.mask_type == 0) {
            n_ctx = n_ctx < 0 ? 0 : n_ctx;
            n_tgt = n_tgt < 0 ? 0 : (n_tgt > sk ? sk : n_tgt);
        }
        const int delta = sk - sq;
        const int hist_k = sk - n_tgt;

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
        const int wr0 = wave * kShortWaveM;
        const bool wave_active = wr0 < sq;

        // ---- K and V rows -> LDS: load instruction i of a tile fills its bytes [1024 i, + 1024), 16 bytes per lane;
        // piece 64 i + lane is row piece / CPR, physical chunk piece % CPR, which holds the logical chunk the swizzle
        // names (XOR swizzles are their own inverse).  Rows past the sequence and chunks past the head dim read as zeros.
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const int instr = WAVES * i + wave;
            const int piece = instr * 64 + lane;
            const int r = piece / CPR;
            const int pc = piece % CPR;
            const int kc = tiny_swizzle<D>(r, pc);
            const int vc = kc;
            const uint32_t k_src = (kc * 8 < a.d_qk) ? static_cast<uint32_t>(r) * k_stride + kc * 16u : kOutOfRange;
            const uint32_t v_src = (vc * 8 < a.d_v) ? static_cast<uint32_t>(r) * v_stride + vc * 16u : kOutOfRange;
            request_to_lds_b128(k_rsrc, lds_address(s_k) + instr * 1024u, k_src);
            request_to_lds_b128(v_rsrc, lds_address(s_v) + instr * 1024u, v_src);
        }
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

        // ---- per-row visibility: visible(j) = j < lim && !(hole_lo <= j < hole_hi) ----
        int row = wr0 + n;
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
        // no row of this wavefront sees a key from here on (the largest limit of its rows)
        int lim_wave = lim;
#pragma unroll
        for (int m = 1; m < 16; m <<= 1) {
            const int other = __shfl_xor(lim_wave, m);
            lim_wave = lim_wave > other ? lim_wave : other;
        }
        lim_wave = uniform(lim_wave);
        // bounds relative to the lane's first key (key = c0 + 16 j + 4 g + r)
        const int lim_lane = lim - 4 * g;
        const int hole_lo_lane = hole_lo - 4 * g;
        const int hole_hi_lane = hole_hi - 4 * g;

        // everything asked for is in (mine, then everybody's)
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt((0 & 15) | (7 << 4) | (15 << 8));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);

        f32x4_t o_acc[MTILES];
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
            o_acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
        if (wave_active) {
            const float c_exp = a.c_exp;
            // the transposing read hands lane i of a 16-lane group column i of the 4 x 16 block whose 8-byte pieces the
            // group's lanes name -- keys 4 g .. 4 g + 3 (+ 16 for the second read)
            const int vr = 4 * g + (n >> 2);
            const int v_row_off = vr * D + 4 * (n & 1);
            const int v_chunk_lo = (n & 3) >> 1;
#pragma unroll
            for (int kb32 = 0; kb32 < ROWS / 32; ++kb32) {
                const int c0 = 32 * kb32;
                if (c0 < lim_wave) {  // (some row of this wavefront sees a key of the block)
                    // S^T (32 keys x 16 rows) = K . Q^T: two blocks of 16 keys
                    f32x4_t s0 = {0.f, 0.f, 0.f, 0.f};
                    f32x4_t s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int js = 0; js < KSTEPS; ++js) {
                        const int off = (c0 + n) * D + tiny_swizzle<D>(n, 4 * js + g) * 8;
                        const u32x4_t ka = *reinterpret_cast<const u32x4_t*>(s_k + off);
                        const u32x4_t kb = *reinterpret_cast<const u32x4_t*>(s_k + off + 16 * D);
                        s0 = mfma16<Tag>(ka, qf[js], s0);
                        s1 = mfma16<Tag>(kb, qf[js], s1);
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
#pragma unroll
                    for (int mt = 0; mt < MTILES; ++mt) {
                        const uint16_t* const vp = s_v + c0 * D + v_row_off + tiny_swizzle<D>(vr, 2 * mt + v_chunk_lo) * 8;
                        const u32x2_t lo = lds_read_tr16_b64(vp);
                        const u32x2_t hi = lds_read_tr16_b64(vp + 16 * D);
                        const u32x4_t va = {lo[0], lo[1], hi[0], hi[1]};
                        o_acc[mt] = mfma16<Tag>(va, pb, o_acc[mt]);
                    }
                }
            }
        }

        // ---- store O: lane (n, g) holds dims 16 mt + 4 g + 0..3 of query row wr0 + n ----
        const float c_out = a.c_out;
        if (a.out_vec_ok != 0) {
            // (everybody is done reading K before anybody writes its rows there)
            __syncthreads();
            uint16_t* const stage = s_k + wave * (16 * D);
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
            constexpr int RPI = 64 / CPR;    // rows per store instruction
            constexpr int kNonTemporal = 2;  // the rows are not read again by this kernel
            const int rr = lane / CPR;
            const int cc = lane % CPR;
#pragma unroll
            for (int i = 0; i < kShortWaveM / RPI; ++i) {
                const int r = i * RPI + rr;
                const u32x4_t piece = *reinterpret_cast<const u32x4_t*>(stage + r * D + (cc ^ (r & (CPR - 1))) * 8);
                const uint32_t off = (cc * 8 < a.d_v) ? static_cast<uint32_t>(wr0 + r) * o_stride + cc * 16u : kOutOfRange;
                __builtin_amdgcn_raw_buffer_store_b128(piece, o_rsrc, static_cast<int>(off), 0, kNonTemporal);
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

    // ---- rows past the last offset belong to no sequence: zero-fill (all workgroups share the job) ----
    {
        const int64_t first_tail = last_offset < 0 ? 0 : (last_offset < a.total_q ? last_offset : a.total_q);
        const int64_t row_elems = static_cast<int64_t>(a.n_heads_q) * a.d_v;
        const int64_t n_tail = (a.total_q - first_tail) * row_elems;
        uint16_t* tail = out16 + first_tail * row_elems;
        for (int64_t e = static_cast<int64_t>(blockIdx.x) * THREADS + tid; e < n_tail;
             e += static_cast<int64_t>(gridDim.x) * THREADS) {
            tail[e] = 0;
        }
    }
}

}  // namespace hstu
