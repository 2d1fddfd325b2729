// HSTU jagged attention backward for gfx950 (MI355X): device code.
//
//   X = alpha (Q K^T + rab),  sig = sigmoid(X),  P = X sig scale M
//   dV = P^T dO,   dP = dO V^T,   dS = alpha scale M dP sig (1 + X (1 - sig)),   d rab = dS,
//   dQ = dS K,     dK = dS^T Q
// (ascendc/attention/hstu_v1/hstu_backward_v1/op_kernel/vector_score.h:159-205; golden
//  ascendc/attention/hstu_v2/test/pytest/backend/ascend_native_backend.py:86-150)
//
// Two kernels, no atomics, every output row written by exactly one wavefront (bitwise reproducible):
//
//   hstu_bwd_dkv_kernel  two workgroups per 128-key tile of one (sequence, K/V head), one per output.  The key rows
//                        stay in registers (B operands) while the query rows that can see them stream through
//                        LDS, 32 at a time, for every query head of the group.  Both outputs in one wavefront
//                        would need 328 registers (one wavefront per SIMD, which cannot overlap its own MFMA and
//                        VALU phases); as two workgroups either fits in 256 and two of them share a CU without
//                        sharing a barrier, so that their phases drift apart and overlap:
//                          dV workgroup:  S = Q . K^T,  P,            dV^T += dO^T . P
//                          dK workgroup:  S = Q . K^T,  dP = dO . V^T,  dS,  dK^T += Q^T . dS
//                        (A operands from LDS: Q, dO plain; dO^T, Q^T by transposed reads; B operands: K, V rows in
//                        registers, P / dS straight from the accumulators)
//   hstu_bwd_dq_kernel   one workgroup per 128-row query tile of one (sequence, head), the forward's shape: Q and
//                        dO rows in registers, K and V sub-tiles stream through LDS.  Per sub-tile:
//                            S^T  = K . Q^T,   dP^T = V . dO^T,   dQ^T += K^T . dS^T
//                        and d rab = dS is stored from the accumulators when asked for.
//
// As in the forward, the score block is computed with the streamed operand as rows, so that its accumulator layout
// (lane = resident row, registers = streamed rows) is the B-operand layout of the products that consume it: P and
// dS never leave registers.  A sub-tile that is read both plainly and transposed is kept in LDS once, in a layout
// that is free of bank conflicts for both reads.  Recomputing S and dP in both kernels costs 7 products instead of 5 and buys
// freedom from atomics and from a dQ workspace (8 with the S computed by both wavefronts of a key set).
#pragma once
#include "hstu_fwd_kernel.hip.h"
#include "hstu_clear.hip.h"

namespace hstu {


struct SeqInfo {
    int64_t q0;
    int64_t k0;
    int sq;
    int sk;
    int n_ctx;
    int n_tgt;
    int delta;
    int hist_k;
};

__device__ __forceinline__ SeqInfo load_seq(const BwdArgs& a, int b)
{
    SeqInfo s;
    int64_t q0 = load_index_uniform(a.offs_q, b, a.idx64);
    int64_t q1 = load_index_uniform(a.offs_q, b + 1, a.idx64);
    int64_t k0 = load_index_uniform(a.offs_k, b, a.idx64);
    int64_t k1 = load_index_uniform(a.offs_k, b + 1, a.idx64);
    q1 = q1 < a.total_q ? q1 : a.total_q;
    k1 = k1 < a.total_k ? k1 : a.total_k;
    q0 = q0 < 0 ? 0 : q0;
    k0 = k0 < 0 ? 0 : k0;
    int sq = static_cast<int>(q1 > q0 ? q1 - q0 : 0);
    int sk = static_cast<int>(k1 > k0 ? k1 - k0 : 0);
    s.sq = sq < a.max_q ? sq : a.max_q;
    s.sk = sk < a.max_k ? sk : a.max_k;
    s.q0 = q0;
    s.k0 = k0;
    s.n_ctx = 0;
    s.n_tgt = 0;
    if (a.mask_type == 0) {
        if (a.num_ctx) {
            s.n_ctx = static_cast<int>(load_index_uniform(a.num_ctx, b, a.idx64));
        }
        if (a.num_tgt) {
            s.n_tgt = static_cast<int>(load_index_uniform(a.num_tgt, b, a.idx64));
        }
        s.n_ctx = s.n_ctx < 0 ? 0 : s.n_ctx;
        s.n_tgt = s.n_tgt < 0 ? 0 : (s.n_tgt > s.sk ? s.sk : s.n_tgt);
    }
    s.delta = s.sk - s.sq;
    s.hist_k = s.sk - s.n_tgt;
    return s;
}

// The longest sequence of the batch in query rows, clamped as load_seq clamps: one pass of the wavefront over the offsets.
// The host sizes the grids of the query-tile kernels from max_seq_len_q, a bound that callers often set far above their
// sequences (a configuration constant); the kernels take the number of tile levels that exist from here, so that the
// workgroups of levels no sequence has come last in the grid instead of first and the heaviest tiles start at once.
__device__ __forceinline__ int batch_max_rows(const BwdArgs& a, int lane)
{
    int longest = 0;
    for (int b = lane; b < a.n_batch; b += 64) {
        int64_t q0 = load_index(a.offs_q, b, a.idx64);
        int64_t q1 = load_index(a.offs_q, b + 1, a.idx64);
        q1 = q1 < a.total_q ? q1 : a.total_q;
        q0 = q0 < 0 ? 0 : q0;
        const int sq = static_cast<int>(q1 > q0 ? q1 - q0 : 0);
        longest = sq > longest ? sq : longest;
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        const int other = __shfl_xor(longest, m, 64);
        longest = other > longest ? other : longest;
    }
    longest = uniform(longest);
    return longest < a.max_q ? longest : a.max_q;
}
// tile levels (of `rows` query rows each) that some sequence of the batch has: at most the host's count, at least one
__device__ __forceinline__ int live_levels(const BwdArgs& a, int lane, int rows, int host_levels)
{
    const int n = (batch_max_rows(a, lane) + rows - 1) / rows;
    return n < 1 ? 1 : (n < host_levels ? n : host_levels);
}

// Slot `slot` of a grid over (tile level, pair) -> its level and pair (`pair` may come out at or past n_pairs: a slot of
// the rounded-up grid that has no work).  Level after level, all pairs of the heaviest level first, keeps the end of a
// launch short -- but the workgroups resident at any time then belong to as many pairs as there are, and once the K / V (or
// Q / dO) rows of all pairs together no longer fit the caches every one of them streams its rows from memory.  Pair after
// pair (a.pair_major; the host's choice for launches of many items over more rows than the caches hold): workgroups go to
// the 8 XCDs in turn, so slot i belongs to XCD i mod 8; XCD x takes the pairs x, x + 8, ... one after the other, the levels
// of a pair next to each other, heaviest first, so that the tiles of a pair run side by side on one XCD and find its rows
// in that XCD's L2.  (The host sizes such a grid as n_levels x 8 x ceil(n_pairs / 8) slots.)
__device__ __forceinline__ void slot_of(const BwdArgs& a, int slot, int n_levels, int n_pairs, int& lvl, int& pair)
{
    if (a.pair_major == 0) {
        lvl = slot / n_pairs;
        pair = slot - lvl * n_pairs;
        return;
    }
    const int j = slot >> 3;
    const int turn = j / n_levels;
    lvl = j - turn * n_levels;
    pair = turn * 8 + (slot & 7);
}

// The pair plane of the 16-bit kernels: what the query-tile kernel hands to the key-tile workgroups of the next launch.
// One 128-byte line per query row and 32-key block: the block's 32 dS values, then its 32 P values.  Lines are packed
// per head by global query row (offs_q[b] + r; no room for rows that the batch does not have), the lines of a row side by
// side -- all ceil(max_k / 32) blocks of it (at a pitch of pair_full_pitch_lines() lines), or, for a causal mask over equal query and key offsets without context
// rows (plane_tri; the host knows this much without reading the offsets), only the blocks 0 .. G that rows of the
// sequence's 32-row group G can see.  The host sizes the triangular form without knowing the lengths: 32 rows of slack
// per sequence make ((offs_q[b] + 32 b) (n_blk + 1) + 1) / 2 lines an upper bound of what the sequences ahead of b hold.
__device__ __forceinline__ int64_t pair_lines_ahead(const BwdArgs& a, int64_t q0, int b)
{
    const int64_t n_blk = (a.max_k + 31) / 32;
    return a.plane_tri ? ((q0 + 32 * static_cast<int64_t>(b)) * (n_blk + 1) + 1) / 2 : q0 * pair_full_pitch_lines(a.max_k);
}
// first byte of sequence b's lines for head h, and their extent
__device__ __forceinline__ uint8_t* pair_plane_of(const BwdArgs& a, int64_t q0, int b, int h)
{
    return static_cast<uint8_t*>(a.p_plane) + (static_cast<int64_t>(h) * a.plane_head_lines + pair_lines_ahead(a, q0, b)) * 128;
}
__device__ __forceinline__ uint32_t pair_seq_bytes(const BwdArgs& a, int sq)
{
    const uint32_t groups = static_cast<uint32_t>(sq + 31) >> 5;
    const uint32_t pitch = static_cast<uint32_t>(pair_full_pitch_lines(a.max_k));
    return (a.plane_tri ? 16u * groups * (groups + 1u) : static_cast<uint32_t>(sq) * pitch) * 128u;
}
// byte offset, from the sequence's first line, of row r's line for block 0
__device__ __forceinline__ uint32_t pair_row_offset(const BwdArgs& a, int r)
{
    const uint32_t g = static_cast<uint32_t>(r) >> 5;
    const uint32_t pitch = static_cast<uint32_t>(pair_full_pitch_lines(a.max_k));
    return (a.plane_tri ? 16u * g * (g + 1u) + (static_cast<uint32_t>(r) & 31u) * (g + 1u) : static_cast<uint32_t>(r) * pitch) * 128u;
}

// Windows (head dims above 256 on the kernels of the slot 256): the real head of head h of a launch, its K/V head, and
// the [max_q][max_k] plane of an attn_bias-shaped tensor for sequence b and head h, in elements
__device__ __forceinline__ int real_head(const BwdArgs& a, int h) { return a.win == 2 ? h >> 1 : h; }
__device__ __forceinline__ int kv_head_of(const BwdArgs& a, int h)
{
    return a.win == 2 ? ((h >> 1) / a.head_ratio) * 2 + (h & 1) : h / a.head_ratio;
}
__device__ __forceinline__ int64_t bias_plane_of(const BwdArgs& a, int b, int h)
{
    return (static_cast<int64_t>(b) * (a.n_heads_q / a.win) + real_head(a, h)) * a.max_q * static_cast<int64_t>(a.max_k);
}
// S and dP of the first window (PHASE 1 of the query-tile kernel writes, PHASE 2 reads): per real head, global query row,
// 32-key block and half-wave the 16 + 16 fp32 accumulator values of the lane, 128 bytes
__device__ __forceinline__ float* partial_of(const BwdArgs& a, int h, int64_t row, int x, int lh)
{
    const int64_t n_blk = (a.max_k + 31) / 32;
    return a.partial + (((static_cast<int64_t>(real_head(a, h)) * a.total_q + row) * n_blk + x) * 2 + lh) * 32;
}

// The one statement of which 32-key blocks the query-tile kernels sweep for the 32 query rows from r0 on (r0 a multiple of
// 32): those that start below this limit.  What such a kernel hands over through a workspace (dS, dS and P) it writes for
// exactly these blocks, and the key-tile kernels read exactly these: both sides, 16-bit and fp32, take the limit from here,
// so a workspace needs no clearing.  (The limit is that of the group's last row, or of its context rows; it never passes
// the sequence's last key.  Rows and 16-byte pieces past the sequence are left out by both sides on top of it.)
__device__ __forceinline__ int swept_key_limit(const BwdArgs& a, const SeqInfo& s, int r0)
{
    return wave_bounds(a.mask_type, r0, s.sq, s.sk, s.n_ctx, s.n_tgt, a.target_group, r0 < s.sq, kWaveM).lim_max;
}

// rows past the last offset belong to no sequence: zero-fill them (all workgroups of a launch share the job)
__device__ __forceinline__ void zero_tail_rows(void* out, const void* offs, int n_batch, int idx64, int64_t total,
                                               int64_t row_elems, int threads)
{
    const int64_t last = load_index_uniform(offs, n_batch, idx64);
    const int64_t first_tail = last < 0 ? 0 : (last < total ? last : total);
    const int64_t n_tail = (total - first_tail) * row_elems;
    uint16_t* const tail = static_cast<uint16_t*>(out) + first_tail * row_elems;
    for (int64_t e = static_cast<int64_t>(blockIdx.x) * threads + threadIdx.x; e < n_tail;
         e += static_cast<int64_t>(gridDim.x) * threads) {
        tail[e] = 0;
    }
}

// first key hidden from query row r by the causal / context rule, and the hole the grouped targets cut out
__device__ __forceinline__ void row_bounds(const SeqInfo& s, int mask_type, int group, int r, int& lim, int& hole_lo,
                                           int& hole_hi)
{
    hole_lo = 0;
    hole_hi = 0;
    if (mask_type != 0) {
        lim = s.sk;
        return;
    }
    lim = r + s.delta + 1;
    if (r < s.n_ctx) {
        lim = lim > s.hist_k ? lim : s.hist_k;
    }
    lim = lim < 0 ? 0 : (lim > s.sk ? s.sk : lim);
    if (s.n_tgt > 0 && group > 0) {
        const int ti = r - (s.sq - s.n_tgt);
        if (ti >= 0) {
            hole_lo = s.hist_k;
            hole_hi = s.hist_k + (ti / group) * group;
        }
    }
}

// The score algebra of the backward, per element, with X = alpha s, sig = sigmoid(X), t = exp(-X):
//   P  = X sig scale                       = s * [alpha scale sig]
//   dS = alpha scale dP sig (1 + X (1 - sig)) = dP * [alpha scale sig] * (1 + s * [alpha (1 - sig)])
// The constants ride on the reciprocal: alpha scale sig = rcp((1 + t) / (alpha scale)) = rcp(fma(t, ci, ci)), and
// alpha (1 - sig) = alpha - [alpha scale sig] / scale.  That is 3 vector instructions and the two transcendental
// ones for P, 6 and two for dS (9 and 8 written out term by term) -- the vector unit is what the steps of these
// kernels wait for as much as the matrix pipe.  alpha = 0 gives P = dS = 0 (ci = inf, rcp(inf) = 0), as it must.
struct ScoreConsts {
    float c_exp;      // -alpha log2(e)
    float ci;         // 1 / (alpha scale)
    float inv_scale;  // 1 / scale
    float alpha;
};
__device__ __forceinline__ ScoreConsts score_consts(float alpha, float scale)
{
    ScoreConsts c;
    c.c_exp = -alpha * 1.4426950408889634f;
    c.ci = 1.0f / (alpha * scale);
    c.inv_scale = 1.0f / scale;
    c.alpha = alpha;
    return c;
}
// alpha scale sigmoid(alpha s)
__device__ __forceinline__ float scaled_sigmoid(float s, const ScoreConsts& c)
{
    const float t = __builtin_amdgcn_exp2f(s * c.c_exp);
    return __builtin_amdgcn_rcpf(__builtin_fmaf(t, c.ci, c.ci));
}
// P (without mask)
__device__ __forceinline__ float score_p(float s, const ScoreConsts& c) { return s * scaled_sigmoid(s, c); }
// dS (without mask)
__device__ __forceinline__ float score_ds(float s, float dp, const ScoreConsts& c)
{
    const float sg = scaled_sigmoid(s, c);
    const float u = __builtin_fmaf(-sg, c.inv_scale, c.alpha);  // alpha (1 - sig)
    return dp * (sg * __builtin_fmaf(s, u, 1.0f));
}

// ---------------------------------------------------------------------------------------------------------
// shared pieces of the two kernels: the two LDS layouts of a 32-row sub-tile and their read patterns
// ---------------------------------------------------------------------------------------------------------
// One LDS layout of a 32-row sub-tile that is free of bank conflicts for both ways it is read here: plainly (A
// operand rows = tile rows: 16 consecutive rows, one 16-byte chunk each) and transposed (ds_read_b64_tr_b16: rows
// 4 h .. 4 h + 3, 64 bytes each).  The XOR term is a bijection of the row bits that index the rows sharing 16 chunk
// positions, with the two bits that tell rows 0..3 apart moved to the top, where they select the 64-byte group.
// Adding 8 to the row flips bit 1 of the term, adding 16 leaves it alone.
template <int D>
__device__ __forceinline__ int both_ways_swizzle(int row, int chunk)
{
    static_assert(D == 64 || D == 128 || D == 256, "layouts exist for 64, 128 and 256 elements per row");
    if constexpr (D >= 128) {  // (a row of 256 elements is two bank sweeps: only the low four chunk bits matter)
        return chunk ^ (((row & 3) << 2) | ((row >> 2) & 3));
    } else {
        const int p = row >> 1;
        return chunk ^ (((p & 1) << 2) | ((p >> 1) & 3));
    }
}

template <int D>
struct SubTile {
    static constexpr int CPR = D / 8;                 // 16-byte chunks per row
    static constexpr int ELEMS = 32 * D;              // 16-bit elements
    static constexpr int KIB = 32 * D * 2 / 1024;     // 1 KiB load instructions per sub-tile
    static constexpr int LPW = KIB >= 4 ? KIB / 4 : 1;  // ... per loading wavefront
    static constexpr int NLW = KIB >= 4 ? 4 : KIB;      // wavefronts that take part
    static constexpr int KSTEPS = D / 16;
    static constexpr int MTILES = D / 32;
};

// The 32 rows x D columns a wavefront holds in MFMA accumulator layout (lane (ln, lh): row ln, columns
// 32 mt + 8 g + 4 lh .. + 3), rounded to the 16-bit type, passed through the wavefront's own 32 x D elements of LDS
// (16-byte chunks XOR-ed with the row) and written 16 bytes per lane: every store instruction writes whole 128-byte
// lines, where storing the accumulators as they lie writes every line in eight pieces.  `first_row_off` = byte
// offset of the tile's row 0 under `rsrc`, whose bound drops rows past the end of the sequence.
template <typename Tag, int D>
__device__ __forceinline__ void store_tile_rows(uint16_t* stage, const f32x16_t (&acc)[D / 32], const __amdgpu_buffer_rsrc_t rsrc,
                                                uint32_t first_row_off, uint32_t stride, int dim_limit, int lane)
{
    constexpr int CPR = D / 8;  // 16-byte chunks per row
    // opaque copy of the lane id: the LDS offsets depend on the lane only, and worked out ahead of the sweep they
    // would take two dozen registers through it
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    const int ln = lane_e & 31, lh = lane_e >> 5;
#pragma unroll
    for (int mt = 0; mt < D / 32; ++mt) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            u32x2_t w;
            w[0] = pack2<Tag>(acc[mt][4 * g + 0], acc[mt][4 * g + 1]);
            w[1] = pack2<Tag>(acc[mt][4 * g + 2], acc[mt][4 * g + 3]);
            const int chunk = (4 * mt + g) ^ (ln & (CPR - 1));
            *reinterpret_cast<u32x2_t*>(stage + ln * D + chunk * 8 + 4 * lh) = w;
        }
    }
    // (one wavefront: its LDS accesses execute in order; the fences keep the compiler from moving the reads up)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    constexpr int RPI = 64 / CPR;  // rows per store instruction
    constexpr int kNonTemporal = 2;  // cache policy bit nt: the rows are not read again by this kernel
    const int rr = lane_e / CPR, cc = lane_e % CPR;
#pragma unroll
    for (int i = 0; i < 32 / RPI; ++i) {
        const int r = i * RPI + rr;
        const u32x4_t piece = *reinterpret_cast<const u32x4_t*>(stage + r * D + (cc ^ (r & (CPR - 1))) * 8);
        const uint32_t off = (cc * 8 < dim_limit) ? first_row_off + static_cast<uint32_t>(r) * stride + cc * 16u : kOutOfRange;
        __builtin_amdgcn_raw_buffer_store_b128(piece, rsrc, static_cast<int>(off), 0, kNonTemporal);
    }
}

// ---------------------------------------------------------------------------------------------------------
// dQ (and d rab)
// ---------------------------------------------------------------------------------------------------------
// STORE: 0 = dQ only; 1 = dS stored as well (it is the attn_bias gradient; or into a workspace, for dK workgroups that
// read it back); 2 = dS and P stored (P for dV workgroups that read it back: no product is then computed twice)
// PHASE (head dims above 256, two windows per head): 0 = everything in one launch.  1 = first window: S and dP of the
// window go to a.partial in fp32, nothing else is written.  2 = second window: S and dP start from a.partial, then as
// PHASE 0 (the dQ written is that of this window).  3 = dQ of the first window from the dS that PHASE 2 stored in the pair
// plane: no scores are computed.
template <typename Tag, int D, bool HAS_RAB, bool HAS_MASK, int STORE, int PHASE = 0>
__global__ __launch_bounds__(256, bwd_dq_wgs_per_cu(D, HAS_RAB, HAS_MASK)) void hstu_bwd_dq_kernel(const BwdArgs a)
{
    static_assert(PHASE == 0 || D == 256, "windows run on the kernels of the slot 256");
    static_assert(PHASE != 1 || STORE == 0, "the first window stores its partial scores only");
    static_assert(PHASE != 3 || STORE == 0, "dQ from the plane stores dQ only");
    constexpr bool WANT_DRAB = STORE >= 1;
    constexpr bool WANT_P = STORE == 2;
    typedef SubTile<D> T;
    constexpr int LPW = T::LPW, NLW = T::NLW, KSTEPS = T::KSTEPS, MTILES = T::MTILES, NCH = 2 * T::MTILES;
    // three stages of {K, V} sub-tiles; separate arrays so that the compiler can tell the stage being filled by
    // the asynchronous loads from the one being read.  K is read plainly (S^T) and transposed (dQ^T) from one copy.
    __shared__ __attribute__((aligned(1024))) uint16_t s_k0[T::ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_k1[T::ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_k2[T::ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v0[T::ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v1[T::ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v2[T::ELEMS];
    // The sub-tile of step x is requested two steps ahead; a wavefront may have the requests of one later step
    // outstanding when it starts a step (requests past the last sub-tile are sent out of range, so that the count
    // per step is constant).  Memory latency under load is longer than one step.
    constexpr int kReqs = 2 * LPW;
    constexpr int kWaitStage = (kReqs & 15) | (7 << 4) | (15 << 8) | ((kReqs >> 4) << 14);
    constexpr uint32_t kPastEnd = 0x40000000u;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = uniform(tid >> 6);
    const int ln = lane & 31;
    const int lh = lane >> 5;

    // heaviest (last) query tiles first
    if constexpr (STORE == 2) {
        if (a.drab_clear_bytes > 0) {
            // (the order in which the dK workgroups of the next launch write the attn_bias gradient: cleared here,
            // beside this kernel's work, by all workgroups alike)
            clear_share(a.drab, a.drab_clear_bytes, blockIdx.x, gridDim.x, threadIdx.x, 256);
        }
    }
    const int grid_heads = a.win_only >= 0 ? a.n_heads_q / a.win : a.n_heads_q;
    const int per_level = a.n_batch * grid_heads;
    int lvl, rem;
    slot_of(a, static_cast<int>(blockIdx.x), a.n_qtiles, per_level, lvl, rem);
    // (heaviest tiles first, counted from the highest level that exists in the batch; with context rows the first tile of a
    // sequence sweeps all of its history keys and goes ahead)
    const int n_levels = live_levels(a, lane, kBlockM, a.n_qtiles);
    const int qt = (a.mask_type == 0 && a.num_ctx != nullptr) ? (lvl == 0 ? 0 : n_levels - lvl) : n_levels - 1 - lvl;
    const int b = rem / grid_heads;
    const int h_grid = rem - b * grid_heads;
    const int h = a.win_only >= 0 ? h_grid * a.win + a.win_only : h_grid;
    const int hk = kv_head_of(a, h);
    if constexpr (PHASE != 1) {
        zero_tail_rows(a.dq, a.offs_q, a.n_batch, a.idx64, a.total_q, static_cast<int64_t>(a.n_heads_q) * a.d_qk, 256);
    }
    if (lvl >= n_levels || rem >= per_level) {
        return;  // a level that no sequence of the batch has, or a slot past the last pair
    }
    const SeqInfo sq_info = load_seq(a, b);
    const int sq = sq_info.sq, sk = sq_info.sk;
    const int r0 = qt * kBlockM;
    if (r0 >= sq) {
        return;
    }
    const int wr0 = r0 + wave * kWaveM;

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
    const __amdgpu_buffer_rsrc_t k_rsrc =
        make_rsrc(static_cast<const uint8_t*>(a.k) + (sq_info.k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_qk) * 2,
                  sk > 0 ? static_cast<uint32_t>(sk - 1) * k_stride + a.d_qk * 2u : 0u);
    const __amdgpu_buffer_rsrc_t v_rsrc =
        make_rsrc(static_cast<const uint8_t*>(a.v) + (sq_info.k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_v) * 2,
                  sk > 0 ? static_cast<uint32_t>(sk - 1) * v_stride + a.d_v * 2u : 0u);

    // per-lane source offsets of the sub-tile loads (see the forward kernel: 16-byte slot -> row, swizzled chunk)
    uint32_t k_src[LPW], v_src[LPW];
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
        const int slot = (wave * LPW + i) * 64 + lane;
        const int r = (slot / T::CPR) & 31;
        const int pc = slot % T::CPR;
        const int cs = both_ways_swizzle<D>(r, pc);  // (its own inverse)
        k_src[i] = (cs * 8 < a.d_qk) ? static_cast<uint32_t>(r) * k_stride + cs * 16u : kOutOfRange;
        v_src[i] = (cs * 8 < a.d_v) ? static_cast<uint32_t>(r) * v_stride + cs * 16u : kOutOfRange;
    }
    int n_lane_off[KSTEPS];  // plain read of row ln, MFMA step js
    int t_lane_off[MTILES][2];  // transposed read, output tile mt: rows vr0 (+ 16 j2) and vr0 + 8 (+ 16 j2)
#pragma unroll
    for (int js = 0; js < KSTEPS; ++js) {
        n_lane_off[js] = ln * D + both_ways_swizzle<D>(ln, 2 * js + lh) * 8;
    }
    {
        const int vr0 = 4 * lh + ((lane & 15) >> 2);
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
            const int col = 32 * mt + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
            t_lane_off[mt][0] = vr0 * D + both_ways_swizzle<D>(vr0, col >> 3) * 8 + (col & 7);
            t_lane_off[mt][1] = (vr0 + 8) * D + both_ways_swizzle<D>(vr0 + 8, col >> 3) * 8 + (col & 7);
        }
    }

    // keys needed by this tile (as in the forward)
    int kmax;
    if (a.mask_type == 0) {
        const int r1 = (r0 + kBlockM < sq) ? r0 + kBlockM : sq;
        kmax = r1 + sq_info.delta;
        if (r0 < sq_info.n_ctx) {
            kmax = kmax > sq_info.hist_k ? kmax : sq_info.hist_k;
        }
        kmax = kmax < 0 ? 0 : (kmax > sk ? sk : kmax);
    } else {
        kmax = sk;
    }
    const int n_sub = (kmax + 31) / 32;

    // resident rows: Q and dO fragments (B operands: lane = row, 8 dims per MFMA step)
    u32x4_t qf[KSTEPS], gf[KSTEPS];
    {
        const uint32_t q_off = static_cast<uint32_t>(wr0 + ln) * q_stride;
        const uint32_t g_off = static_cast<uint32_t>(wr0 + ln) * g_stride;
#pragma unroll
        for (int js = 0; js < KSTEPS; ++js) {
            const int d0 = 16 * js + 8 * lh;
            qf[js] = __builtin_amdgcn_raw_buffer_load_b128(q_rsrc, static_cast<int>(d0 < a.d_qk ? q_off + d0 * 2u : kOutOfRange), 0, 0);
            gf[js] = __builtin_amdgcn_raw_buffer_load_b128(g_rsrc, static_cast<int>(d0 < a.d_v ? g_off + d0 * 2u : kOutOfRange), 0, 0);
        }
    }
    int row = wr0 + ln;
    row = row < sq - 1 ? row : sq - 1;
    int lim, hole_lo, hole_hi;
    row_bounds(sq_info, a.mask_type, a.target_group, row, lim, hole_lo, hole_hi);
    const WaveBounds wb = wave_bounds(a.mask_type, wr0, sq, sk, sq_info.n_ctx, sq_info.n_tgt, a.target_group, wr0 < sq);
    const int nx_w = (swept_key_limit(a, sq_info, wr0) + 31) / 32;  // (= wb.lim_max: a wavefront is a 32-row group here)
    // Context rows: the keys [row_only_lo, row_only_hi) lie past the limit of every row of this wavefront that is not a
    // context row and below the limit of each of its context rows (and before the target keys, when target rows carve
    // holes): a row sees a sub-tile in that range whole or not at all -- nearly every step of a sequence's first tile.
    int row_only_lo = 0, row_only_hi = 0;
    if (a.mask_type == 0 && wr0 < sq && wr0 < sq_info.n_ctx) {
        const int wr1 = (wr0 + kWaveM < sq) ? wr0 + kWaveM : sq;
        int other_hi = sq_info.n_ctx < wr1 ? wr1 + sq_info.delta : 0;
        other_hi = other_hi < 0 ? 0 : (other_hi > sk ? sk : other_hi);
        int ctx_lo = wr0 + sq_info.delta + 1 > sq_info.hist_k ? wr0 + sq_info.delta + 1 : sq_info.hist_k;
        ctx_lo = (wb.any_hole && ctx_lo > sq_info.hist_k) ? sq_info.hist_k : ctx_lo;
        ctx_lo = ctx_lo < 0 ? 0 : (ctx_lo > sk ? sk : ctx_lo);
        row_only_lo = uniform(other_hi);
        row_only_hi = uniform(ctx_lo);
    }

    const uint32_t bias_bytes = static_cast<uint32_t>(a.max_q) * static_cast<uint32_t>(a.max_k) * 2u;
    const int64_t bias_plane = bias_plane_of(a, b, h);
    const __amdgpu_buffer_rsrc_t rab_rsrc =
        make_rsrc(HAS_RAB ? static_cast<const uint16_t*>(a.rab) + bias_plane : nullptr, HAS_RAB ? bias_bytes : 0u);
    const __amdgpu_buffer_rsrc_t mask_rsrc =
        make_rsrc(HAS_MASK ? static_cast<const uint16_t*>(a.mask) + bias_plane : nullptr, HAS_MASK ? bias_bytes : 0u);
    const __amdgpu_buffer_rsrc_t drab_rsrc =
        make_rsrc(WANT_DRAB ? static_cast<uint16_t*>(a.drab) + bias_plane : nullptr, WANT_DRAB ? bias_bytes : 0u);
    // dS and P together (STORE 2) go to the pair plane: one whole 128-byte line per row and step, where two planes of the
    // bias layout would each get half a line
    const __amdgpu_buffer_rsrc_t p_rsrc =
        make_rsrc((WANT_P || PHASE == 3) ? pair_plane_of(a, sq_info.q0, b, real_head(a, h)) : nullptr,
                  (WANT_P || PHASE == 3) ? pair_seq_bytes(a, sq) : 0u);
    const uint32_t pair_row_off = ((WANT_P || PHASE == 3) && wr0 + ln < sq) ? pair_row_offset(a, wr0 + ln) : kOutOfRange;
    // rows past the sequence lie inside the plane but must stay untouched / unread: their offset leaves it
    const uint32_t bias_row_off =
        (wr0 + ln < sq) ? static_cast<uint32_t>(wr0 + ln) * static_cast<uint32_t>(a.max_k) * 2u : kOutOfRange;
    const bool vec = a.bias_vec_ok != 0;
    const bool vec16 = a.bias_vec_ok == 2;  // rab / mask / d rab rows are 16-byte aligned

    // words 2g, 2g+1 = the row's values at keys c0 + 8g + 4 lh + 0..3 (accumulator order)
    auto load_words = [&](__amdgpu_buffer_rsrc_t rsrc, int c0, uint32_t (&w)[8]) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int key = c0 + 8 * g + 4 * lh;
            const uint32_t off = bias_row_off + static_cast<uint32_t>(key) * 2u;
            if (vec) {
                const U32Pair t = __builtin_bit_cast(
                    U32Pair, __builtin_amdgcn_raw_buffer_load_b64(rsrc, static_cast<int>(key < a.max_k ? off : kOutOfRange), 0, 0));
                w[2 * g + 0] = t.v[0];
                w[2 * g + 1] = t.v[1];
            } else {
                uint32_t e[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    uint32_t eoff = (key + i < a.max_k) ? off + 2u * i : kOutOfRange;
                    asm volatile("" : "+v"(eoff));
                    e[i] = __builtin_amdgcn_raw_buffer_load_b16(rsrc, static_cast<int>(eoff), 0, 0);
                }
                w[2 * g + 0] = (e[0] & 0xffffu) | (e[1] << 16);
                w[2 * g + 1] = (e[2] & 0xffffu) | (e[3] << 16);
            }
        }
    };

    f32x16_t dq_acc[MTILES];
#pragma unroll
    for (int mt = 0; mt < MTILES; ++mt) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            dq_acc[mt][i] = 0.f;
        }
    }
    const ScoreConsts sconst = score_consts(a.alpha, a.scale);

    static_assert(NLW == 4, "every wavefront takes part in the loads");
    auto request = [&](uint16_t* kd, uint16_t* vd, int x) {
        {
            const uint32_t kb = x < n_sub ? static_cast<uint32_t>(x * 32) * k_stride : kPastEnd;
            const uint32_t vb = x < n_sub ? static_cast<uint32_t>(x * 32) * v_stride : kPastEnd;
#pragma unroll
            for (int i = 0; i < LPW; ++i) {
                load_to_lds_b128(k_rsrc, kd + (wave * LPW + i) * 512, k_src[i] + kb);
                load_to_lds_b128(v_rsrc, vd + (wave * LPW + i) * 512, v_src[i] + vb);
            }
        }
    };
    auto read_n = [&](const uint16_t* tile, int js) -> u32x4_t {
        return *reinterpret_cast<const u32x4_t*>(tile + n_lane_off[js]);
    };
    auto read_t = [&](const uint16_t* tile, int c) -> u32x4_t {
        const int j2 = c / MTILES, mt = c % MTILES;
        const u32x2_t lo = lds_read_tr16_b64(tile + t_lane_off[mt][0] + 16 * j2 * D);
        const u32x2_t hi = lds_read_tr16_b64(tile + t_lane_off[mt][1] + 16 * j2 * D);
        const u32x4_t r = {lo[0], lo[1], hi[0], hi[1]};
        return r;
    };

    auto step = [&](const uint16_t* kn, const uint16_t* vn, uint16_t* kn_o, uint16_t* vn_o, int x) {
        // sub-tile x has landed (mine, then everybody's), and nobody reads the stage of step x - 1 any more: all
        // LDS reads of a step feed MFMAs that were issued before the barrier.  (A bare barrier: __syncthreads()
        // would add a fence that waits for every outstanding request.)
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(kWaitStage);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        // rab / mask values of this step go out before the tile requests: loads return in order, so waiting for
        // them then only waits for requests of earlier steps, not for the ones made now
        const int c0 = x * 32;
        uint32_t rw[8], mw[8];
        f32x16_t s, dp;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            s[i] = 0.f;
            dp[i] = 0.f;
        }
        uint32_t pk[8];
        uint32_t pp[8];  // P, when it is stored
        if (x < nx_w) {
            if constexpr (HAS_RAB && PHASE != 1 && PHASE != 3) {
                load_words(rab_rsrc, c0, rw);
            }
            if constexpr (HAS_MASK && PHASE != 1 && PHASE != 3) {
                load_words(mask_rsrc, c0, mw);
            }
            if constexpr (PHASE == 2) {
                // the sums over the first window: where the accumulators start
                if (wr0 + ln < sq) {
                    const float4* const from = reinterpret_cast<const float4*>(partial_of(a, h, sq_info.q0 + wr0 + ln, x, lh));
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float4 t = from[i], u = from[4 + i];
                        s[4 * i + 0] = t.x, s[4 * i + 1] = t.y, s[4 * i + 2] = t.z, s[4 * i + 3] = t.w;
                        dp[4 * i + 0] = u.x, dp[4 * i + 1] = u.y, dp[4 * i + 2] = u.z, dp[4 * i + 3] = u.w;
                    }
                }
            }
            if constexpr (PHASE == 3) {
                // dS of this step as PHASE 2 stored it: the lane pair of a row holds 16-byte pieces (keys 16 h2 + 8 lh .. + 7)
                // and trades halves back into accumulator order (the swap is its own inverse); pieces that start past the
                // last key were not written and read as zeros
                typedef __attribute__((ext_vector_type(2))) unsigned u2_t;
#pragma unroll
                for (int h2 = 0; h2 < 2; ++h2) {
                    const int key = c0 + 16 * h2 + 8 * lh;
                    const uint32_t off = pair_row_off + static_cast<uint32_t>(2 * c0 + 16 * h2 + 8 * lh) * 2u;
                    const U32Quad wd = __builtin_bit_cast(
                        U32Quad, __builtin_amdgcn_raw_buffer_load_b128(p_rsrc, static_cast<int>(key < sk ? off : kOutOfRange), 0, 0));
                    const u2_t d0 = __builtin_amdgcn_permlane32_swap(wd.v[0], wd.v[2], false, false);
                    const u2_t d1 = __builtin_amdgcn_permlane32_swap(wd.v[1], wd.v[3], false, false);
                    pk[4 * h2 + 0] = d0[0];
                    pk[4 * h2 + 2] = d0[1];
                    pk[4 * h2 + 1] = d1[0];
                    pk[4 * h2 + 3] = d1[1];
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        request(kn_o, vn_o, x + 2);
        __builtin_amdgcn_sched_barrier(0);
        if (x >= nx_w) {
            return;  // nothing of this sub-tile is visible to the rows of this wavefront
        }
        if constexpr (PHASE != 3) {
#pragma unroll
            for (int js = 0; js < KSTEPS; ++js) {
                s = mfma32<Tag>(read_n(kn, js), qf[js], s);
                dp = mfma32<Tag>(read_n(vn, js), gf[js], dp);
            }
        }
        if constexpr (PHASE == 1) {
            if (wr0 + ln < sq) {
                float4* const to = reinterpret_cast<float4*>(partial_of(a, h, sq_info.q0 + wr0 + ln, x, lh));
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    to[i] = make_float4(s[4 * i + 0], s[4 * i + 1], s[4 * i + 2], s[4 * i + 3]);
                    to[4 + i] = make_float4(dp[4 * i + 0], dp[4 * i + 1], dp[4 * i + 2], dp[4 * i + 3]);
                }
            }
            return;
        }
        if constexpr (PHASE != 3) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float ds2[2], p2[2];
#pragma unroll
            for (int e2 = 0; e2 < 2; ++e2) {
                const int e = 2 * i + e2;
                float sv = s[e];
                if constexpr (HAS_RAB) {
                    sv += e2 ? hi_to_float<Tag>(rw[i]) : lo_to_float<Tag>(rw[i]);
                }
                float ds = score_ds(sv, dp[e], sconst);
                float pv = WANT_P ? score_p(sv, sconst) : 0.f;
                if constexpr (HAS_MASK) {
                    const float mv = e2 ? hi_to_float<Tag>(mw[i]) : lo_to_float<Tag>(mw[i]);
                    ds *= mv;
                    pv *= mv;
                }
                ds2[e2] = ds;
                p2[e2] = pv;
            }
            pk[i] = pack2<Tag>(ds2[0], ds2[1]);
            if constexpr (WANT_P) {
                pp[i] = pack2<Tag>(p2[0], p2[1]);
            }
        }
        // visibility, applied to the packed values and only when the sub-tile is not fully visible to this
        // wavefront's rows (as in the forward): key c0 + 8 (e / 4) + 4 lh + e % 4 of element e is hidden at or past
        // lim and inside the hole
        const bool full = (c0 + 32 <= wb.lim_min) && !(wb.any_hole && c0 + 32 > sq_info.hist_k && c0 < wb.hole_hi_max);
        if (!full && c0 >= row_only_lo && c0 + 32 <= row_only_hi) {
            const uint32_t keep = lim > c0 ? 0xffffffffu : 0u;  // (a context row's limit is at or past c0 + 32, any other row's at or before c0)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                pk[i] &= keep;
                if constexpr (WANT_P) {
                    pp[i] &= keep;
                }
            }
        } else if (!full) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                uint32_t keep = 0;
#pragma unroll
                for (int e2 = 0; e2 < 2; ++e2) {
                    const int e = 2 * i + e2;
                    const int key = c0 + 8 * (e / 4) + 4 * lh + (e % 4);
                    const bool vis = (key < lim) && !(key >= hole_lo && key < hole_hi);
                    keep |= vis ? (0xffffu << (16 * e2)) : 0u;
                }
                pk[i] &= keep;
                if constexpr (WANT_P) {
                    pp[i] &= keep;
                }
            }
        }
        }  // PHASE != 3
        if constexpr (WANT_P) {
            // the two lanes of a row trade halves (see below), then four 16-byte pieces per lane pair: dS, dS, P, P
            typedef __attribute__((ext_vector_type(2))) unsigned u2_t;
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2) {
                const int key = c0 + 16 * h2 + 8 * lh;
                const uint32_t off = pair_row_off + static_cast<uint32_t>(2 * c0 + 16 * h2 + 8 * lh) * 2u;
                const u2_t d0 = __builtin_amdgcn_permlane32_swap(pk[4 * h2 + 0], pk[4 * h2 + 2], false, false);
                const u2_t d1 = __builtin_amdgcn_permlane32_swap(pk[4 * h2 + 1], pk[4 * h2 + 3], false, false);
                const u32x4_t wd = {d0[0], d1[0], d0[1], d1[1]};
                __builtin_amdgcn_raw_buffer_store_b128(wd, p_rsrc, static_cast<int>(key < sk ? off : kOutOfRange), 0, 0);
                const u2_t r0 = __builtin_amdgcn_permlane32_swap(pp[4 * h2 + 0], pp[4 * h2 + 2], false, false);
                const u2_t r1 = __builtin_amdgcn_permlane32_swap(pp[4 * h2 + 1], pp[4 * h2 + 3], false, false);
                const u32x4_t wp = {r0[0], r1[0], r0[1], r1[1]};
                __builtin_amdgcn_raw_buffer_store_b128(wp, p_rsrc, static_cast<int>(key < sk ? off + 64u : kOutOfRange), 0, 0);
            }
        }
        if constexpr (WANT_DRAB && !WANT_P) {
            if (vec16) {
                // 16-byte aligned rows: the two lanes of a row trade halves (v_permlane32_swap), so that each holds 8
                // consecutive keys and a store instruction writes whole 32-byte sectors of 32 rows instead of 16-byte
                // pieces.  Lane (row, 0) ends up with keys 16 h2 + 0..7, lane (row, 1) with keys 16 h2 + 8..15.
                typedef __attribute__((ext_vector_type(2))) unsigned u2_t;
#pragma unroll
                for (int h2 = 0; h2 < 2; ++h2) {
                    const u2_t r0 = __builtin_amdgcn_permlane32_swap(pk[4 * h2 + 0], pk[4 * h2 + 2], false, false);
                    const u2_t r1 = __builtin_amdgcn_permlane32_swap(pk[4 * h2 + 1], pk[4 * h2 + 3], false, false);
                    const u32x4_t w4 = {r0[0], r1[0], r0[1], r1[1]};
                    const int key = c0 + 16 * h2 + 8 * lh;
                    const uint32_t off = bias_row_off + static_cast<uint32_t>(key) * 2u;
                    __builtin_amdgcn_raw_buffer_store_b128(w4, drab_rsrc, static_cast<int>(key < sk ? off : kOutOfRange), 0, 0);
                }
            } else {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int key = c0 + 8 * g + 4 * lh;
                    const uint32_t off = bias_row_off + static_cast<uint32_t>(key) * 2u;
                    if (vec) {
                        const u32x2_t w2 = {pk[2 * g], pk[2 * g + 1]};
                        __builtin_amdgcn_raw_buffer_store_b64(w2, drab_rsrc, static_cast<int>(key < sk ? off : kOutOfRange), 0, 0);
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const uint32_t word = pk[2 * g + i / 2];
                            const uint16_t val = static_cast<uint16_t>((i & 1) ? (word >> 16) : (word & 0xffffu));
                            __builtin_amdgcn_raw_buffer_store_b16(val, drab_rsrc,
                                                                  static_cast<int>(key + i < sk ? off + 2u * i : kOutOfRange), 0, 0);
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int j2 = c / MTILES, mt = c % MTILES;
            const u32x4_t pb = {pk[4 * j2 + 0], pk[4 * j2 + 1], pk[4 * j2 + 2], pk[4 * j2 + 3]};
            dq_acc[mt] = mfma32<Tag>(read_t(kn, c), pb, dq_acc[mt]);
        }
    };

    if (n_sub > 0) {
        request(s_k0, s_v0, 0);
        request(s_k1, s_v1, 1);
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

    if constexpr (PHASE == 1) {
        return;
    }
    // store dQ: lane holds query row (wr0 + ln), dims 32*mt + 8*g + 4*lh + 0..3
    if (a.grad_vec_ok != 0) {
        // (every wavefront is done with the ring before anybody writes its rows into a stage)
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        uint16_t* const stage = wave == 0 ? s_k0 : (wave == 1 ? s_k1 : (wave == 2 ? s_k2 : s_v0));
        store_tile_rows<Tag, D>(stage, dq_acc, dq_rsrc, static_cast<uint32_t>(wr0) * q_stride, q_stride, a.d_qk, lane);
    } else {
        const uint32_t row_off = static_cast<uint32_t>(wr0 + ln) * q_stride;
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d0 = 32 * mt + 8 * g + 4 * lh;
                const uint32_t off = (d0 < a.d_qk) ? row_off + d0 * 2u : kOutOfRange;
                u32x2_t w;
                w[0] = pack2<Tag>(dq_acc[mt][4 * g + 0], dq_acc[mt][4 * g + 1]);
                w[1] = pack2<Tag>(dq_acc[mt][4 * g + 2], dq_acc[mt][4 * g + 3]);
                __builtin_amdgcn_raw_buffer_store_b64(w, dq_rsrc, static_cast<int>(off), 0, 0);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------------
// dK, dV
// ---------------------------------------------------------------------------------------------------------

// MODE 0: a dV and a dK workgroup per key tile (8 apart in the grid, see below).  MODE 1 and 2 serve the three-launch order
// dV / dQ / dK: all workgroups of a launch have one role, and the dK ones (MODE 2; rab and mask play no part in it)
// take dS from the attn_bias gradient that the query-tile kernel wrote between the two launches.
// MODE 4: launched after a query-tile kernel that stored dS and P: a workgroup that takes dV from P and one that
// takes dK from dS per key tile, both of MODE 2's build (one product each; the dV ones stream dO where the dK ones
// stream Q).  MODE 5: the same, and the dK workgroups write the dS pieces they read into the attn_bias gradient, which
// the query-tile kernel cleared beside its work: the order for a call that wants that gradient.
template <typename Tag, int D, bool HAS_RAB, bool HAS_MASK, int MODE = 0>
__global__ __launch_bounds__(kDkvThreads, (MODE == 2 || MODE >= 4) ? bwd_dk_from_ds_wgs_per_cu(D) : bwd_dkv_wgs_per_cu(D, HAS_RAB, HAS_MASK)) void hstu_bwd_dkv_kernel(const BwdArgs a)
{
    typedef SubTile<D> T;
    constexpr int LPW = T::LPW, NLW = T::NLW, KSTEPS = T::KSTEPS, MTILES = T::MTILES, NCH = 2 * T::MTILES;
    constexpr int kHalves = (MODE == 2 || MODE >= 4) ? 1 : 2;  // (a workgroup that reads dS or P streams Q or dO only)
    // four stages, each the Q sub-tile followed by the dO sub-tile (separate arrays per stage, see the dQ kernel;
    // Q and dO of a stage share an array so that a wavefront can address "the tile of my role" by an offset)
    __shared__ __attribute__((aligned(1024))) uint16_t s_st0[kHalves * T::ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_st1[kHalves * T::ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_st2[kHalves * T::ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_st3[kHalves * T::ELEMS];
    // a sub-tile is requested three steps ahead: the requests of two later steps may be outstanding at a step's start
    // (plus, where dS / P rows are read, the two loads of the next step's rows, issued between the two requests.  Reading rab / mask
    // rows a step ahead in the same way was tried for the other modes: nothing for the dV-only launch, 277 -> 314 us
    // at C3 for the two-role one, which has no registers to spare at the head-dim slot 128.)
    constexpr int kAhead = (MODE == 2 || MODE >= 4) ? 2 : 0;  // (MODE 5's stores only make the wait stricter: the count must hold from the first step on)
    constexpr int kReqs = 2 * kHalves * LPW + kAhead;
    constexpr int kWaitStage = (kReqs & 15) | (7 << 4) | (15 << 8) | ((kReqs >> 4) << 14);
    constexpr uint32_t kPastEnd = 0x40000000u;
    static_assert(NLW == 4, "every wavefront takes part in the loads");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = uniform(tid >> 6);
    // In the launches with both roles the dV and the dK workgroup of a key tile are 8 apart in the grid: workgroups go
    // to the 8 XCDs in turn, so the two land on one XCD and find each other's Q / dO rows (MODE 0), or the other half of
    // every line of the dS / P plane (MODE 4), in its L2.  (The host rounds the grid up to whole groups of 16; the
    // slots past the last tile leave below like those of absent tiles.)
    constexpr bool from_plane = MODE == 2 || MODE >= 4;
    constexpr bool paired = MODE == 0 || MODE >= 4;
    const bool dk_role = paired ? ((blockIdx.x >> 3) & 1) != 0 : MODE == 2;
    const int ln = lane & 31;
    const int lh = lane >> 5;

    // key tile 0 is seen by the most query rows: heaviest first
    const int per_level = a.n_batch * a.n_heads_k;
    const int tile_slot = static_cast<int>(paired ? (blockIdx.x >> 4) * 8 + (blockIdx.x & 7) : blockIdx.x);
    int kt_idx, rem;
    slot_of(a, tile_slot, a.n_ktiles, per_level, kt_idx, rem);
    const int b = rem / a.n_heads_k;
    const int hk = rem - b * a.n_heads_k;
    if constexpr (MODE != 1) {
        zero_tail_rows(a.dk, a.offs_k, a.n_batch, a.idx64, a.total_k, static_cast<int64_t>(a.n_heads_k) * a.d_qk, kDkvThreads);
    }
    if constexpr (MODE != 2) {
        zero_tail_rows(a.dv, a.offs_k, a.n_batch, a.idx64, a.total_k, static_cast<int64_t>(a.n_heads_k) * a.d_v, kDkvThreads);
    }
    if (a.drab_clear_bytes > 0) {
        // the attn_bias gradient is cleared here, by all workgroups alike (also those of absent tiles, which leave
        // below), and written by the query-tile kernel that runs after this one.  (Dealing the share out over the
        // steps of the sweep instead, a few stores per thread and step, was measured slower: stores and tile
        // requests retire through one in-order counter.)
        clear_share(a.drab, a.drab_clear_bytes, blockIdx.x, gridDim.x, tid, kDkvThreads);
    }
    if (rem >= per_level) {
        return;  // (pair after pair: a slot past the last pair)
    }
    const SeqInfo si = load_seq(a, b);
    const int sq = si.sq, sk = si.sk;
    const int c0 = kt_idx * kBlockM;
    if (c0 >= sk) {
        return;
    }
    const int cw0 = c0 + wave * 32;  // first key of this wavefront
    const int key = cw0 + ln;        // this lane's key

    const uint32_t q_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_qk * 2u;
    const uint32_t g_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_v * 2u;
    const uint32_t k_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_qk * 2u;
    const uint32_t v_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_v * 2u;
    const __amdgpu_buffer_rsrc_t k_rsrc =
        make_rsrc(static_cast<const uint8_t*>(a.k) + (si.k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_qk) * 2,
                  static_cast<uint32_t>(sk - 1) * k_stride + a.d_qk * 2u);
    const __amdgpu_buffer_rsrc_t v_rsrc =
        make_rsrc(static_cast<const uint8_t*>(a.v) + (si.k0 * a.n_heads_k + hk) * static_cast<int64_t>(a.d_v) * 2,
                  static_cast<uint32_t>(sk - 1) * v_stride + a.d_v * 2u);
    // the output of this wavefront's role
    const uint32_t out_stride = dk_role ? k_stride : v_stride;
    const int out_dim = dk_role ? a.d_qk : a.d_v;
    const __amdgpu_buffer_rsrc_t out_rsrc =
        make_rsrc(static_cast<uint8_t*>(dk_role ? a.dk : a.dv) + (si.k0 * a.n_heads_k + hk) * static_cast<int64_t>(out_dim) * 2,
                  static_cast<uint32_t>(sk - 1) * out_stride + static_cast<uint32_t>(out_dim) * 2u);

    // per-lane source offsets of the sub-tile loads (Q into the first half of a stage, dO into the second)
    uint32_t q_src[LPW], g_src[LPW];
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
        const int slot = (wave * LPW + i) * 64 + lane;
        const int r = (slot / T::CPR) & 31;
        const int pc = slot % T::CPR;
        const int cs = both_ways_swizzle<D>(r, pc);
        q_src[i] = (cs * 8 < a.d_qk) ? static_cast<uint32_t>(r) * q_stride + cs * 16u : kOutOfRange;
        g_src[i] = (cs * 8 < a.d_v) ? static_cast<uint32_t>(r) * g_stride + cs * 16u : kOutOfRange;
    }
    int n_lane_off[KSTEPS];
    int t_lane_off[MTILES][2];
#pragma unroll
    for (int js = 0; js < KSTEPS; ++js) {
        n_lane_off[js] = ln * D + both_ways_swizzle<D>(ln, 2 * js + lh) * 8;
    }
    {
        const int vr0 = 4 * lh + ((lane & 15) >> 2);
        // the transposed operand of this role: Q^T (first half of a stage) for dK, dO^T (second half) for dV
        const int role_half = (dk_role || from_plane) ? 0 : T::ELEMS;  // (a stage of one half holds the role's tile)
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
            const int col = 32 * mt + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
            t_lane_off[mt][0] = role_half + vr0 * D + both_ways_swizzle<D>(vr0, col >> 3) * 8 + (col & 7);
            t_lane_off[mt][1] = role_half + (vr0 + 8) * D + both_ways_swizzle<D>(vr0 + 8, col >> 3) * 8 + (col & 7);
        }
    }

    // resident rows: K (both roles) and V (dK role) fragments of this lane's key
    u32x4_t kf[KSTEPS], vf[KSTEPS];
    {
        const uint32_t k_off = static_cast<uint32_t>(key) * k_stride;
        const uint32_t v_off = static_cast<uint32_t>(key) * v_stride;
#pragma unroll
        for (int js = 0; js < KSTEPS; ++js) {
            const int d0 = 16 * js + 8 * lh;
            kf[js] = __builtin_amdgcn_raw_buffer_load_b128(k_rsrc, static_cast<int>(d0 < a.d_qk ? k_off + d0 * 2u : kOutOfRange), 0, 0);
            vf[js] = __builtin_amdgcn_raw_buffer_load_b128(v_rsrc, static_cast<int>(dk_role && !from_plane && d0 < a.d_v ? v_off + d0 * 2u : kOutOfRange), 0, 0);
        }
    }

    // query sub-tiles that can see a key of this tile
    // (causal: from the sub-tile of the first row that sees key c0 on; with context rows ahead of that, which see every history
    // key: their sub-tiles first, then the same -- the sub-tiles in between see nothing of this tile and are skipped)
    const int n_qsub = (sq + 31) / 32;
    int x_first = 0;
    int x_skip_from = -1, x_skip_to = -1;
    if (a.mask_type == 0) {
        const int first_row = c0 - si.delta;  // the first row that sees key c0
        const int x_causal = first_row > 0 ? first_row / 32 : 0;
        if (si.n_ctx > 0 && c0 < si.hist_k) {
            const int ctx_end = ((si.n_ctx < sq ? si.n_ctx : sq) + 31) / 32;  // sub-tiles that hold context rows
            if (x_causal > ctx_end) {
                x_skip_from = ctx_end;
                x_skip_to = x_causal < n_qsub ? x_causal : n_qsub;
            }
        } else {
            x_first = x_causal;
        }
    }
    const int nx = (n_qsub > x_first ? n_qsub - x_first : 0) - (x_skip_to - x_skip_from);
    const int n_iter = nx * a.head_ratio;  // (query head of the group, query sub-tile), head-major

    f32x16_t acc[MTILES];  // dK^T or dV^T of this wavefront's keys, by role
#pragma unroll
    for (int mt = 0; mt < MTILES; ++mt) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            acc[mt][i] = 0.f;
        }
    }
    const ScoreConsts sconst = score_consts(a.alpha, a.scale);
    const uint32_t bias_bytes = static_cast<uint32_t>(a.max_q) * static_cast<uint32_t>(a.max_k) * 2u;
    const bool targets = a.mask_type == 0 && si.n_tgt > 0 && a.target_group > 0;
    // rab / custom mask tiles are wanted with lane = key and registers = query rows, but lie in memory with the
    // keys of a query row side by side.  With 16-byte aligned rows they are read the way they lie (lane = query
    // row, 8 consecutive keys per 16-byte load) as the A operand of two MFMAs whose B operand is a constant 0/1
    // matrix that routes k-slot (half lh, element e) of MFMA j to key column 16 j + 8 lh + e: the matrix pipe does
    // the transposition (exactly: every product is a value times 1 or 0), and rab lands in the S accumulators.
    // With rows that start at multiples of 8 bytes only (max_seq_len_k a multiple of 4, not of 8) a piece of 8 keys is
    // two 8-byte loads, and its second half is asked for only when it starts inside the row (inside the sequence's keys,
    // for values that another kernel wrote piece by piece): past it lies the next row.
    const bool vec16 = a.bias_vec_ok == 2;
    const bool vec8 = a.bias_vec_ok != 0;
    auto load_piece = [&](const __amdgpu_buffer_rsrc_t rsrc, uint32_t off, bool second_half) -> u32x4_t {
        if (vec16) {
            return __builtin_amdgcn_raw_buffer_load_b128(rsrc, static_cast<int>(off), 0, 0);
        }
        const u32x2_t lo = __builtin_amdgcn_raw_buffer_load_b64(rsrc, static_cast<int>(off), 0, 0);
        const u32x2_t hi = __builtin_amdgcn_raw_buffer_load_b64(rsrc, static_cast<int>(second_half ? off + 8u : kOutOfRange), 0, 0);
        const u32x4_t r = {lo[0], lo[1], hi[0], hi[1]};
        return r;
    };
    u32x4_t route[2] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
    if constexpr (HAS_RAB || HAS_MASK || from_plane) {
        const uint32_t one = std::is_same<Tag, bf16_tag>::value ? 0x3f80u : 0x3c00u;  // 1.0 in the input type
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int d = ln - 16 * j - 8 * lh;  // the element of this lane's k-slots that is 1, if in 0..7
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                route[j][i] = (d == 2 * i) ? one : (d == 2 * i + 1) ? (one << 16) : 0u;
            }
        }
    }

    // head and sub-tile of iteration it, kept incrementally (no division in the loop)
    // (windows: K/V head hk is window hk % win of the real K/V head hk / win; its query heads follow win apart)
    const int first_h = (hk / a.win) * a.head_ratio * a.win + (hk % a.win);
    int req_h = first_h, req_x = x_first, req_it = 0;  // next request
    int cur_h = first_h, cur_x = x_first;              // current step
    auto request = [&](uint16_t* stage) {
        const bool past = req_it >= n_iter;  // (sent out of range: moves no data, keeps the count per step constant)
        const __amdgpu_buffer_rsrc_t q_rsrc =
            make_rsrc(static_cast<const uint8_t*>(a.q) + (si.q0 * a.n_heads_q + req_h) * static_cast<int64_t>(a.d_qk) * 2,
                      static_cast<uint32_t>(sq - 1) * q_stride + a.d_qk * 2u);
        const __amdgpu_buffer_rsrc_t g_rsrc =
            make_rsrc(static_cast<const uint8_t*>(a.grad) + (si.q0 * a.n_heads_q + req_h) * static_cast<int64_t>(a.d_v) * 2,
                      static_cast<uint32_t>(sq - 1) * g_stride + a.d_v * 2u);
        const uint32_t qb = past ? kPastEnd : static_cast<uint32_t>(req_x * 32) * q_stride;
        const uint32_t gb = past ? kPastEnd : static_cast<uint32_t>(req_x * 32) * g_stride;
#pragma unroll
        for (int i = 0; i < LPW; ++i) {
            if constexpr (from_plane) {
                if (dk_role) {
                    load_to_lds_b128(q_rsrc, stage + (wave * LPW + i) * 512, q_src[i] + qb);
                } else {
                    load_to_lds_b128(g_rsrc, stage + (wave * LPW + i) * 512, g_src[i] + gb);
                }
            } else {
                load_to_lds_b128(q_rsrc, stage + (wave * LPW + i) * 512, q_src[i] + qb);
                load_to_lds_b128(g_rsrc, stage + T::ELEMS + (wave * LPW + i) * 512, g_src[i] + gb);
            }
        }
        ++req_it;
        if (++req_x == x_skip_from) {
            req_x = x_skip_to;
        }
        if (req_x >= n_qsub) {
            req_x = x_first;
            if (!past && req_it < n_iter) {
                req_h += a.win;
            }
        }
    };
    auto read_n = [&](const uint16_t* tile, int js) -> u32x4_t {
        return *reinterpret_cast<const u32x4_t*>(tile + n_lane_off[js]);
    };
    auto read_t = [&](const uint16_t* stage, int c) -> u32x4_t {
        const int j2 = c / MTILES, mt = c % MTILES;
        const u32x2_t lo = lds_read_tr16_b64(stage + t_lane_off[mt][0] + 16 * j2 * D);
        const u32x2_t hi = lds_read_tr16_b64(stage + t_lane_off[mt][1] + 16 * j2 * D);
        const u32x4_t r = {lo[0], lo[1], hi[0], hi[1]};
        return r;
    };

    // whole block hidden from the keys of this wavefront?  (rows rq0 .. rq0 + 31, keys cw0 .. cw0 + 31)
    auto block_active = [&](int rq0) -> bool { return cw0 < swept_key_limit(a, si, rq0); };
    // MODE 2 and 4: the dS (or P) rows of a step, as the query-tile kernel stored them (rounded to the input type, masked), are
    // read like rab rows -- lane (ln, lh) reads row rq0 + ln, keys cw0 + 16 j + 8 lh .. + 7 -- one step ahead of
    // their use, and transposed by the same routing products.  Only what that kernel wrote is read -- whole 16-byte
    // pieces that start ahead of the sequence's last key, in the 32 x 32 blocks that it swept, which are the active
    // blocks here -- so the plane need not be cleared when it is a workspace.  The two loads go out every step
    // (out of range when there is nothing to read: no data moves), so that the number of requests in flight at the
    // start of a step is the same whatever the blocks are.
    u32x4_t ds_next[2] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
    int ds_steps = 0;  // steps whose dS rows have been asked for
    auto load_ds = [&](int h, int rq0) {
        const bool wanted = ds_steps < n_iter && block_active(rq0);
        ++ds_steps;
        // (MODE 4: dS and P share a plane of their own layout, see the query-tile kernel: per row and 32-key block, 32
        // dS values followed by 32 P values)
        const uint32_t pitch = static_cast<uint32_t>(a.max_k);
        const __amdgpu_buffer_rsrc_t ds_rsrc =
            MODE >= 4 ? make_rsrc(pair_plane_of(a, si.q0, b, real_head(a, h)), pair_seq_bytes(a, sq))
                      : make_rsrc(static_cast<const uint16_t*>(a.drab) + bias_plane_of(a, b, h),
                                  static_cast<uint32_t>(a.max_q) * pitch * 2u);
        const uint32_t row_off = MODE >= 4 ? pair_row_offset(a, rq0 + ln) : static_cast<uint32_t>(rq0 + ln) * pitch * 2u;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int key0 = cw0 + 16 * j + 8 * lh;
            const uint32_t col = MODE >= 4 ? static_cast<uint32_t>(2 * cw0 + 16 * j + 8 * lh + (dk_role ? 0 : 32)) : static_cast<uint32_t>(key0);
            const uint32_t off = (wanted && rq0 + ln < sq && key0 < sk) ? row_off + col * 2u : kOutOfRange;
            if constexpr (MODE >= 4) {  // (the pair plane: 16-byte pieces whatever max_seq_len_k is)
                ds_next[j] = __builtin_amdgcn_raw_buffer_load_b128(ds_rsrc, static_cast<int>(off), 0, 0);
            } else {
                ds_next[j] = load_piece(ds_rsrc, off, key0 + 4 < sk);
            }
        }
    };

    auto step = [&](const uint16_t* stage, uint16_t* stage_o) {
        // this step's sub-tile has landed for everybody; the stage of the previous step is free (see the dQ kernel)
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(kWaitStage);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        const int h = cur_h;
        const int rq0 = cur_x * 32;  // first query row of the sub-tile
        if (++cur_x == x_skip_from) {
            cur_x = x_skip_to;
        }
        if (cur_x >= n_qsub) {
            cur_x = x_first;
            cur_h += a.win;
        }
        const bool active = block_active(rq0);
        const __amdgpu_buffer_rsrc_t rab_rsrc = make_rsrc(
            HAS_RAB ? static_cast<const uint16_t*>(a.rab) + bias_plane_of(a, b, h) : nullptr,
            HAS_RAB ? bias_bytes : 0u);
        const __amdgpu_buffer_rsrc_t mask_rsrc = make_rsrc(
            HAS_MASK ? static_cast<const uint16_t*>(a.mask) + bias_plane_of(a, b, h) : nullptr,
            HAS_MASK ? bias_bytes : 0u);
        // rab / mask rows of this step (16-byte path): lane (ln, lh) has row rq0 + ln, keys cw0 + 16 j + 8 lh .. + 7
        // (whole chunks are in or out of the row: max_seq_len_k is a multiple of 8 here)
        u32x4_t ra[2] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
        u32x4_t ma[2] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
        if constexpr (from_plane) {
            ra[0] = ds_next[0];  // asked for a step ago
            ra[1] = ds_next[1];
            load_ds(cur_h, cur_x * 32);  // (cur_h, cur_x: already those of the next step)
        } else if constexpr (HAS_RAB || HAS_MASK) {
            // (ahead of the tile requests: loads return in order, so waiting for them then only waits for requests
            // of earlier steps)
            if (vec8 && active) {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int key0 = cw0 + 16 * j + 8 * lh;
                    const uint32_t off = (rq0 + ln < sq && key0 < a.max_k)
                                             ? (static_cast<uint32_t>(rq0 + ln) * static_cast<uint32_t>(a.max_k) + static_cast<uint32_t>(key0)) * 2u
                                             : kOutOfRange;
                    if constexpr (HAS_RAB) {
                        ra[j] = load_piece(rab_rsrc, off, key0 + 4 < a.max_k);
                    }
                    if constexpr (HAS_MASK) {
                        ma[j] = load_piece(mask_rsrc, off, key0 + 4 < a.max_k);
                    }
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        request(stage_o);
        if constexpr (MODE == 5) {
            // d rab = dS: the 16-byte pieces just read (row rq0 + ln, keys cw0 + 16 j + 8 lh .. + 7) go to the attn_bias
            // gradient as they are; both stores every step (out of range when there is nothing to write), behind the
            // step's loads, so that no load waits for them
            if (dk_role) {
                const __amdgpu_buffer_rsrc_t drab_rsrc = make_rsrc(
                    static_cast<uint16_t*>(a.drab) + bias_plane_of(a, b, h),
                    bias_bytes);
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int key0 = cw0 + 16 * j + 8 * lh;
                    const uint32_t off = (active && rq0 + ln < sq && key0 < sk)
                                             ? (static_cast<uint32_t>(rq0 + ln) * static_cast<uint32_t>(a.max_k) + static_cast<uint32_t>(key0)) * 2u
                                             : kOutOfRange;
                    if (vec16) {
                        __builtin_amdgcn_raw_buffer_store_b128(ra[j], drab_rsrc, static_cast<int>(off), 0, 0);
                    } else {  // (8-byte pieces; the second one only when it starts inside the sequence's keys)
                        const u32x2_t lo = {ra[j][0], ra[j][1]}, hi = {ra[j][2], ra[j][3]};
                        __builtin_amdgcn_raw_buffer_store_b64(lo, drab_rsrc, static_cast<int>(off), 0, 0);
                        __builtin_amdgcn_raw_buffer_store_b64(hi, drab_rsrc, static_cast<int>(key0 + 4 < sk ? off + 8u : kOutOfRange), 0, 0);
                    }
                }
            } else {
                // (the dV workgroups keep the same count of requests in flight)
                const __amdgpu_buffer_rsrc_t none = make_rsrc(static_cast<uint16_t*>(nullptr), 0u);
                __builtin_amdgcn_raw_buffer_store_b128(ra[0], none, static_cast<int>(kOutOfRange), 0, 0);
                __builtin_amdgcn_raw_buffer_store_b128(ra[1], none, static_cast<int>(kOutOfRange), 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (from_plane) {
          if (active) {
            f32x16_t s;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                s[i] = 0.f;
            }
            s = mfma32<Tag>(ra[0], route[0], s);
            s = mfma32<Tag>(ra[1], route[1], s);
            uint32_t pk[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                pk[i] = pack2<Tag>(s[2 * i], s[2 * i + 1]);  // (exact: the values are of the input type)
            }
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                const int j2 = c / MTILES, mt = c % MTILES;
                const u32x4_t pb = {pk[4 * j2 + 0], pk[4 * j2 + 1], pk[4 * j2 + 2], pk[4 * j2 + 3]};
                acc[mt] = mfma32<Tag>(read_t(stage, c), pb, acc[mt]);
            }
          }
        } else if (active) {
            f32x16_t s, dp;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                s[i] = 0.f;
                dp[i] = 0.f;
            }
            // two independent accumulation chains per wavefront, so that an MFMA never waits for the one before it:
            // S and dP for the dK role; the even and the odd steps of S for the dV role (dp then holds half of S)
            if (dk_role) {
#pragma unroll
                for (int js = 0; js < KSTEPS; ++js) {
                    s = mfma32<Tag>(read_n(stage, js), kf[js], s);
                    dp = mfma32<Tag>(read_n(stage + T::ELEMS, js), vf[js], dp);
                }
            } else {
#pragma unroll
                for (int js = 0; js < KSTEPS; js += 2) {
                    s = mfma32<Tag>(read_n(stage, js), kf[js], s);
                    dp = mfma32<Tag>(read_n(stage, js + 1), kf[js + 1], dp);
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    s[i] += dp[i];
                }
            }
            // fully visible block: every row's lim is past the last key, no context / target effects, all in range
            bool full = (cw0 + 32 <= sk) && (rq0 + 32 <= sq);
            if (a.mask_type == 0) {
                full = full && (cw0 + 32 <= rq0 + si.delta + 1) && !(targets && rq0 + 31 >= sq - si.n_tgt);
            }
            // X and the custom mask value of every element, then the role's own function of it
            float xs[16], ms[16];
            f32x16_t mt16;  // custom mask tile, transposed by the matrix pipe
            if constexpr (HAS_RAB || HAS_MASK) {
                if (vec8) {
                    if constexpr (HAS_RAB) {
                        s = mfma32<Tag>(ra[0], route[0], s);
                        s = mfma32<Tag>(ra[1], route[1], s);
                    }
                    if constexpr (HAS_MASK) {
#pragma unroll
                        for (int i = 0; i < 16; ++i) {
                            mt16[i] = 0.f;
                        }
                        mt16 = mfma32<Tag>(ma[0], route[0], mt16);
                        mt16 = mfma32<Tag>(ma[1], route[1], mt16);
                    }
                }
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int r = rq0 + 8 * (e / 4) + 4 * lh + (e % 4);  // query row of this element
                xs[e] = s[e];
                ms[e] = 1.0f;
                if constexpr (HAS_MASK) {
                    if (vec8) {
                        ms[e] = mt16[e];
                    }
                }
                if constexpr (HAS_RAB || HAS_MASK) {
                    if (!vec8) {
                    const uint32_t boff = (r < sq && key < a.max_k)
                                              ? (static_cast<uint32_t>(r) * static_cast<uint32_t>(a.max_k) + static_cast<uint32_t>(key)) * 2u
                                              : kOutOfRange;
                    if constexpr (HAS_RAB) {
                        const uint32_t raw = __builtin_amdgcn_raw_buffer_load_b16(rab_rsrc, static_cast<int>(boff), 0, 0);
                        xs[e] += lo_to_float<Tag>(raw & 0xffffu);
                    }
                    if constexpr (HAS_MASK) {
                        const uint32_t raw = __builtin_amdgcn_raw_buffer_load_b16(mask_rsrc, static_cast<int>(boff), 0, 0);
                        ms[e] = lo_to_float<Tag>(raw & 0xffffu);
                    }
                    }
                }
            }
            float o[16];
            if (dk_role) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    o[e] = score_ds(xs[e], dp[e], sconst) * ms[e];
                }
            } else {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    o[e] = score_p(xs[e], sconst) * ms[e];  // P = X sig scale, X = alpha (S + rab)
                }
            }
            if (!full) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int r = rq0 + 8 * (e / 4) + 4 * lh + (e % 4);
                    int lim, hole_lo, hole_hi;
                    row_bounds(si, a.mask_type, a.target_group, r, lim, hole_lo, hole_hi);
                    const bool vis = (r < sq) && (key < lim) && !(key >= hole_lo && key < hole_hi);
                    o[e] = vis ? o[e] : 0.f;
                }
            }
            uint32_t pk[8];  // P (dV role) or dS (dK role), B operand of the output product
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                pk[i] = pack2<Tag>(o[2 * i], o[2 * i + 1]);
            }
            // dK^T += Q^T . dS  or  dV^T += dO^T . P: the transposed operand sits in the role's half of the stage
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                const int j2 = c / MTILES, mt = c % MTILES;
                const u32x4_t pb = {pk[4 * j2 + 0], pk[4 * j2 + 1], pk[4 * j2 + 2], pk[4 * j2 + 3]};
                acc[mt] = mfma32<Tag>(read_t(stage, c), pb, acc[mt]);
            }
        }
    };

    if (n_iter > 0) {
        request(s_st0);
        request(s_st1);
        if constexpr (from_plane) {
            load_ds(cur_h, cur_x * 32);  // (where the steps issue theirs: ahead of the request of two stages on)
        }
        request(s_st2);
        int it = 0;
        while (true) {  // (step it reads stage it mod 4 and has stage (it + 3) mod 4 filled)
            step(s_st0, s_st3);
            if (++it >= n_iter) {
                break;
            }
            step(s_st1, s_st0);
            if (++it >= n_iter) {
                break;
            }
            step(s_st2, s_st1);
            if (++it >= n_iter) {
                break;
            }
            step(s_st3, s_st2);
            if (++it >= n_iter) {
                break;
            }
        }
    }

    // store dK or dV: lane holds key (cw0 + ln), dims 32*mt + 8*g + 4*lh + 0..3
    if (a.grad_vec_ok != 0) {
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        uint16_t* const stage = wave == 0 ? s_st0 : (wave == 1 ? s_st1 : (wave == 2 ? s_st2 : s_st3));
        store_tile_rows<Tag, D>(stage, acc, out_rsrc, static_cast<uint32_t>(cw0) * out_stride, out_stride, out_dim, lane);
    } else {
        const uint32_t row_off = static_cast<uint32_t>(key) * out_stride;
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d0 = 32 * mt + 8 * g + 4 * lh;
                u32x2_t w;
                w[0] = pack2<Tag>(acc[mt][4 * g + 0], acc[mt][4 * g + 1]);
                w[1] = pack2<Tag>(acc[mt][4 * g + 2], acc[mt][4 * g + 3]);
                __builtin_amdgcn_raw_buffer_store_b64(w, out_rsrc, static_cast<int>(d0 < out_dim ? row_off + d0 * 2u : kOutOfRange), 0, 0);
            }
        }
    }
}

}  // namespace hstu
