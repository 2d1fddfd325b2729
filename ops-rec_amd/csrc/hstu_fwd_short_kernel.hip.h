// HSTU jagged attention forward for gfx950 (MI355X): the kernel for short work lists.
//
// The persistent kernel (hstu_fwd_kernel.hip.h) gives a wavefront 32 query rows and keeps the matrix pipe and the
// vector ALU busy with a rolling pipeline inside that wavefront; one of its time steps over a 32-key sub-tile takes
// about 0.75 us whether or not anything else runs on the SIMD, so a launch whose list is only an item or two per
// resident workgroup lasts as long as its longest item: (keys / 32) steps one after the other.  This kernel is
// built the other way round for such launches:
//
//   * a wavefront takes 16 query rows (v_mfma_f32_16x16x32), so a step is half the work and half as long, and a
//     workgroup of eight wavefronts covers the same 128-row query tile.  It needs under 128 registers, so four
//     wavefronts share a SIMD (two workgroups per CU) and hide each other's waits: a step is plain code --
//     S^T = K . Q^T, P^T = silu(S^T) masked, O^T += V^T . P^T -- with no pipeline across steps, and a wavefront that
//     has the SIMD to itself at the end of a launch runs faster, not the same;
//   * no work list: one workgroup per (query tile, sequence, head) slot, heaviest tiles first in the grid, the
//     hardware dispatcher balancing them.  A workgroup reads its own four offsets and leaves at once when its tile
//     lies past the end of its sequence, so nothing is sorted, counted or searched before the first product;
//   * slot -> workgroup so that all tiles that read the K / V rows of one (sequence, K/V head) run on one XCD
//     (workgroup i runs on XCD i mod 8) and find those rows in that XCD's L2.
//
// It pays twice the LDS operand traffic per product (an A operand of 1 KiB feeds a 16-row MFMA instead of a 32-row
// one), which is why long lists stay on the persistent kernel.  Same arithmetic per element as that kernel:
// p = s / (1 + exp2(-alpha log2e s)) rounded to the input type, alpha * silu_scale applied once to the fp32 output,
// rows leave as whole 128-byte lines through LDS.  16-bit inputs, built-in mask (causal with context rows, target
// rows and target groups) or no mask, with or without attn_bias (added to the fp32 scores ahead of the SiLU).
//
// What this replaces in the reference (Ascend C): the same pieces as the persistent kernel, with the stream-K split
// of ascendc/attention/hstu_v1/hstu_forward_v1/op_kernel/atlas950/hstu_split_core_policy.h:53-236 answered by
// narrower wavefronts instead of parts of the key range.
#pragma once
#include "hstu_fwd_kernel.hip.h"

namespace hstu {

typedef __attribute__((ext_vector_type(4))) float f32x4_t;

constexpr int kShortWaveM = 16;     // query rows per wavefront
constexpr int kShortWavesPerSimd = 4;  // two workgroups per CU

template <typename Tag>
__device__ __forceinline__ f32x4_t mfma16(u32x4_t a, u32x4_t b, f32x4_t c);
template <>
__device__ __forceinline__ f32x4_t mfma16<bf16_tag>(u32x4_t a, u32x4_t b, f32x4_t c)
{
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                   0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4_t mfma16<f16_tag>(u32x4_t a, u32x4_t b, f32x4_t c)
{
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0,
                                                  0, 0);
}

// V sub-tile in LDS for the 16-row kernel: the transposed read of a half-wave touches rows 4g .. 4g + 3 of two
// neighbouring groups g and the same 32 bytes of each, so 64-byte groups are XOR-ed with the row's low two bits and
// the 32-byte half with its third bit: eight rows x 32 bytes cover all banks once.
template <int D>
__device__ __forceinline__ int v16_chunk_swizzle(int row, int chunk)
{
    static_assert(D == 128, "built for the head-dim slot 128");
    return chunk ^ (((row & 3) << 2) | (((row >> 2) & 1) << 1));
}

// Tile request of the 16-row kernel: 64 lanes x 16 bytes, global -> LDS without passing registers, written as
// assembly so that the compiler's wait-count pass does not see it.  That pass orders a read of an LDS array behind
// the requests it believes may fill that array, and loses track of which is which once there are more request
// instructions than it keeps apart (eight) or a loop's first trip is peeled: it then waits for requests of later
// steps before every read, which undoes the prefetch.  Here the ordering is the kernel's own: a wavefront waits
// for its requests by count (vmcnt) and the workgroup meets at a barrier before a slot is read.  m0 holds the LDS
// address of the wavefront's 1 KiB piece.
__device__ __forceinline__ void request_to_lds_b128(u32x4_t rsrc, uint32_t lds_byte_address, uint32_t voffset)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :
                 : "s"(lds_byte_address), "v"(voffset), "s"(rsrc)
                 : "memory", "m0");
}
__device__ __forceinline__ u32x4_t make_rsrc_words(const void* base, uint32_t bytes)
{
    const uint64_t addr = reinterpret_cast<uint64_t>(base);
    const u32x4_t r = {static_cast<uint32_t>(addr), static_cast<uint32_t>(addr >> 32) & 0xffffu, bytes, kBufferFlags};
    return r;
}
__device__ __forceinline__ uint32_t lds_address(const void* p)
{
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) void*)(p)));
}

// The slot (position in the grid) of a workgroup -> level, (sequence, K/V head) pair and query head of the pair.
// Pairs are padded to a multiple of 8 per level so that pair p lands on XCD p mod 8 at every level: the query tiles
// that read the K / V rows of a pair find them in one L2.  (Measured on lengths 256..1024, batch 32, 4 heads: letting
// the tiles of a pair alternate between two XCDs evens out the XCDs' loads -- with 4 K/V heads XCD x holds head x mod 4
// of every other sequence, and the two halves of a batch of 32 differ by a fifth of the work -- but fetches 135.4 MB
// instead of 77.9 MB for the launch and is no faster once the inputs do not replay out of the memory-side cache.)
struct ShortSlot {
    int level;
    int pair;
    int r;  // query head within the K/V head's group
};
__device__ __forceinline__ ShortSlot short_slot(int idx, int n_pairs, int ratio)
{
    const int pairs_pad = (n_pairs + 7) & ~7;
    const int per_level = pairs_pad * ratio;
    ShortSlot s;
    s.level = div_small(idx, per_level);
    const int in_level = idx - s.level * per_level;
    const int x = in_level & 7;
    const int y = in_level >> 3;
    const int yq = div_small(y, ratio);
    s.r = y - yq * ratio;
    s.pair = yq * 8 + x;
    return s;
}

// attn_bias values for the 16-row kernel, as assembly for the same reason as the tile requests: lane (n, g) asks for
// the four values at keys 4 g .. 4 g + 3 of each 16-key half of a sub-tile of its row (8 bytes each, 32 bytes apart).
// The registers named here are written when the data arrives; rab_wait() is where the kernel makes sure of that.
__device__ __forceinline__ void request_rab(u32x2_t& lo, u32x2_t& hi, u32x4_t rsrc, uint32_t voffset, uint32_t soffset)
{
    asm volatile("buffer_load_dwordx2 %0, %2, %3, %4 offen\n\tbuffer_load_dwordx2 %1, %2, %3, %4 offen offset:32"
                 : "=&v"(lo), "=&v"(hi)
                 : "v"(voffset), "s"(rsrc), "s"(soffset));
}
// waits until at most `open` of this wavefront's memory requests are outstanding; the bias registers pass through
// it so that nothing that reads them moves ahead of the wait
template <int OPEN>
__device__ __forceinline__ void rab_wait(u32x2_t& lo, u32x2_t& hi)
{
    static_assert(OPEN >= 0 && OPEN < 16, "vmcnt fits the low four bits here");
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(lo), "+v"(hi) : "n"(OPEN));
}

template <typename Tag, int D, bool HAS_RAB = false>
__global__ __launch_bounds__(kShortThreads, kShortWavesPerSimd) void hstu_fwd_short_kernel(const FwdArgs a)
{
    static_assert(D == 128, "built for the head-dim slot 128");
    constexpr int SUB_ELEMS = 32 * D;       // one 32-key sub-tile, in 16-bit units
    constexpr int CPR = D / 8;              // 16-byte chunks per row
    constexpr int KSTEPS = D / 32;          // MFMA steps over the head dim (QK product)
    constexpr int MTILES = D / 16;          // 16-wide output tiles over the head dim (PV product)
    constexpr int SUB_KIB = 32 * D * 2 / 1024;  // 1 KiB load instructions per sub-tile: one per wavefront
    static_assert(SUB_KIB == kShortThreads / 64, "one load instruction per wavefront and sub-tile");
    // vmcnt(4): the tile requests of two steps may be open; with a bias the two bias requests of a step come on top
    // (steps t - 1 and t: five pairs since the tile requests of sub-tile t + 1)
    constexpr int kWaitTiles = ((HAS_RAB ? 10 : 4) & 15) | (7 << 4) | (15 << 8);
    constexpr uint32_t kPastEnd = 0x40000000u;

    // four slots each for K and V sub-tiles (sub-tile x in slot x mod 4); separate arrays so that the compiler can
    // tell the slot being filled by the asynchronous loads from the one being read
    __shared__ __attribute__((aligned(1024))) uint16_t s_k0[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_k1[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_k2[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_k3[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v0[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v1[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v2[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v3[SUB_ELEMS];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = uniform(tid >> 6);
    const int n = lane & 15;   // query row of the wavefront / key row of a 16-key block / output dim of a tile
    const int g = lane >> 4;   // which 8 of the 32 contraction values, which 4 of the 16 accumulator rows

    uint16_t* const out16 = static_cast<uint16_t*>(a.out);
    const int n_levels = a.n_qtiles;
    const int ratio = a.head_ratio;
    const int n_pairs = a.n_batch * a.n_heads_k;

#ifdef HSTU_TIMELINE
    uint64_t tl[6] = {__builtin_amdgcn_s_memrealtime(), 0, 0, 0, 0, 0};
#define HSTU_TL(i) tl[i] = __builtin_amdgcn_s_memrealtime()
#else
#define HSTU_TL(i)
#endif
    const int64_t last_offset = load_index_uniform(a.offs_q, a.n_batch, a.idx64);

    // ---- the item of this workgroup ----
    const ShortSlot slot = short_slot(static_cast<int>(blockIdx.x), n_pairs, ratio);
    bool live = slot.pair < n_pairs && slot.level < n_levels;
    int b = 0, hk = 0;
    if (live) {
        b = div_small(slot.pair, a.n_heads_k);
        hk = slot.pair - b * a.n_heads_k;
    }
    const int h = hk * ratio + slot.r;
    // heaviest tiles first; with context rows the first tile of a sequence sweeps all of its history keys, so it goes ahead
    // of the others instead of last
    const bool ctx_first = a.mask_type == 0 && a.num_ctx != nullptr;
    const int qt = ctx_first ? (slot.level == 0 ? 0 : n_levels - slot.level) : n_levels - 1 - slot.level;
    int64_t q0 = 0, q1 = 0, k0 = 0, k1 = 0;
    int n_ctx = 0, n_tgt = 0;
    if (live) {
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
    const int r0 = qt * kBlockM;
    live = live && r0 < sq;

    if (live) {
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

        const int wr0 = r0 + wave * kShortWaveM;
        const bool wave_active = wr0 < sq;  // inactive wavefronts still take part in loads and barriers
        // ---- keys needed by this item ----
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
        const int n_sub = (kmax + 31) / 32;

        // K / V sub-tile streaming: the load instruction of this wavefront fills LDS bytes [wave * 1024, + 1024) of a
        // slot; the per-lane source offset is fixed, only the base moves
        uint32_t k_src, v_src;
        {
            const int piece = wave * 64 + lane;  // 16-byte piece within the sub-tile
            const int r = piece / CPR;
            const int pc = piece % CPR;
            const int kc = k_chunk_swizzle<D>(r, pc);  // XOR swizzles are their own inverse
            const int vc = v16_chunk_swizzle<D>(r, pc);
            k_src = (kc * 8 < a.d_qk) ? static_cast<uint32_t>(r) * k_stride + kc * 16u : kOutOfRange;
            v_src = (vc * 8 < a.d_v) ? static_cast<uint32_t>(r) * v_stride + vc * 16u : kOutOfRange;
        }
        auto k_slot = [&](auto ic) -> uint16_t* {
            constexpr int I = decltype(ic)::value & 3;
            if constexpr (I == 0) {
                return s_k0;
            } else if constexpr (I == 1) {
                return s_k1;
            } else if constexpr (I == 2) {
                return s_k2;
            } else {
                return s_k3;
            }
        };
        auto v_slot = [&](auto ic) -> uint16_t* {
            constexpr int I = decltype(ic)::value & 3;
            if constexpr (I == 0) {
                return s_v0;
            } else if constexpr (I == 1) {
                return s_v1;
            } else if constexpr (I == 2) {
                return s_v2;
            } else {
                return s_v3;
            }
        };
        // requests past the last sub-tile move nothing but keep the number of requests per step constant
        auto request = [&](auto ic, int x) {
            const uint32_t past = (x < n_sub) ? 0u : kPastEnd;
            request_to_lds_b128(k_rsrc, lds_address(k_slot(ic)) + wave * 1024u, k_src + static_cast<uint32_t>(x * 32) * k_stride + past);
            request_to_lds_b128(v_rsrc, lds_address(v_slot(ic)) + wave * 1024u, v_src + static_cast<uint32_t>(x * 32) * v_stride + past);
        };
        typedef std::integral_constant<int, 0> ic0_t;
        typedef std::integral_constant<int, 1> ic1_t;
        typedef std::integral_constant<int, 2> ic2_t;
        typedef std::integral_constant<int, 3> ic3_t;

        HSTU_TL(1);
        // ---- start-up: the first sub-tile, the Q fragment, then two more sub-tiles ----
        // Q fragment (B operand of the first product): lane (n, g) holds Q[row n][32 js + 8 g .. + 7]
        request(ic0_t{}, 0);
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
        request(ic1_t{}, 1);
        request(ic2_t{}, 2);

        // LDS read offsets relative to a sub-tile, in elements.  K operand of MFMA step js: key row n (+ 16 for the
        // second block of 16 keys, same swizzle), chunk 4 js + g.  V^T operand of output tile mt: the transposing read
        // hands lane i of a 16-lane group column i of the 4 x 16 block whose 8-byte pieces the group's lanes name --
        // keys 4 g .. 4 g + 3 (+ 16 for the second read), dims 16 mt .. + 15.
        int k_lane_off[KSTEPS];
#pragma unroll
        for (int js = 0; js < KSTEPS; ++js) {
            k_lane_off[js] = n * D + k_chunk_swizzle<D>(n, 4 * js + g) * 8;
        }
        const int vr = 4 * g + (n >> 2);
        const int v_row_off = vr * D + 4 * (n & 1);
        const int v_chunk_lo = (n & 3) >> 1;  // which 16-byte chunk of the tile's two
        auto v_lane_off = [&](int mt) -> int { return v_row_off + v16_chunk_swizzle<D>(vr, 2 * mt + v_chunk_lo) * 8; };

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
        const WaveBounds wb =
            wave_bounds(a.mask_type, wr0, sq, sk, n_ctx, n_tgt, a.target_group, wave_active, kShortWaveM);
        const int nx_w = (wb.lim_max + 31) / 32;  // sub-tiles this wavefront's rows can see (<= n_sub)
        // bounds relative to the lane's first key of a sub-tile (key = c0 + 16 j + 4 g + r)
        const int lim_lane = lim - 4 * g;
        const int hole_lo_lane = hole_lo - 4 * g;
        const int hole_hi_lane = hole_hi - 4 * g;

        f32x4_t o_acc[MTILES];
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
            o_acc[mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
        const float c_exp = a.c_exp;

        // ---- attn_bias: [batch, heads, max_q, max_k] in the input type; the values of sub-tile x are asked for two steps
        // ahead into one of two register blocks (x & 1).  (Four steps ahead into four blocks: 3 to 8 % slower on every
        // shape measured, 128 registers.)  Requests past the plane of this (sequence, head) read as zeros;
        // those past the row or the sequence read values that the visibility test discards.
        u32x4_t rab_rsrc = {0u, 0u, 0u, 0u};
        uint32_t rab_voff = 0;
        u32x2_t rab_lo0 = {0u, 0u}, rab_hi0 = {0u, 0u}, rab_lo1 = {0u, 0u}, rab_hi1 = {0u, 0u};
        if constexpr (HAS_RAB) {
            const int64_t plane = (static_cast<int64_t>(b) * a.n_heads_q + h) * a.max_q * static_cast<int64_t>(a.max_k);
            rab_rsrc = make_rsrc_words(static_cast<const uint16_t*>(a.rab) + plane,
                                       static_cast<uint32_t>(a.max_q) * static_cast<uint32_t>(a.max_k) * 2u);
            rab_voff = static_cast<uint32_t>(wr0 + n) * static_cast<uint32_t>(a.max_k) * 2u + 8u * g;
            request_rab(rab_lo0, rab_hi0, rab_rsrc, rab_voff, 0u);
            request_rab(rab_lo1, rab_hi1, rab_rsrc, rab_voff, 64u);
        }

        // one step over sub-tile t, which lies in slot S = t mod 4
        auto step = [&](auto sc, const int t) {
            constexpr int S = decltype(sc)::value;
            // the slot of sub-tile t - 1 is free (everybody passed the barrier that ended step t - 1)
            request(std::integral_constant<int, (S + 3) & 3>{}, t + 3);
            if (t < nx_w) {
                const uint16_t* const kt = k_slot(sc);
                const uint16_t* const vt = v_slot(sc);
                const int c0 = t * 32;
                // S^T (32 keys x 16 rows) = K . Q^T: two blocks of 16 keys
                f32x4_t s0 = {0.f, 0.f, 0.f, 0.f};
                f32x4_t s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int js = 0; js < KSTEPS; ++js) {
                    const u32x4_t ka = *reinterpret_cast<const u32x4_t*>(kt + k_lane_off[js]);
                    const u32x4_t kb = *reinterpret_cast<const u32x4_t*>(kt + k_lane_off[js] + 16 * D);
                    s0 = mfma16<Tag>(ka, qf[js], s0);
                    s1 = mfma16<Tag>(kb, qf[js], s1);
                }
                if constexpr (HAS_RAB) {
                    // the bias of this sub-tile is in: asked for two steps ago, and since then the tile requests and the
                    // bias requests of one step and the tile requests of this one have gone out
                    u32x2_t& lo = (S & 1) ? rab_lo1 : rab_lo0;
                    u32x2_t& hi = (S & 1) ? rab_hi1 : rab_hi0;
                    rab_wait<6>(lo, hi);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        s0[e] += (e & 1) ? hi_to_float<Tag>(lo[e >> 1]) : lo_to_float<Tag>(lo[e >> 1]);
                        s1[e] += (e & 1) ? hi_to_float<Tag>(hi[e >> 1]) : lo_to_float<Tag>(hi[e >> 1]);
                    }
                }
                // P^T = silu(S^T), masked, rounded: element (j, r) is key c0 + 16 j + 4 g + r of this lane's row
                float p[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float s = e < 4 ? s0[e] : s1[e - 4];
                    float tt = __builtin_amdgcn_exp2f(s * c_exp);
                    tt = __builtin_amdgcn_rcpf(1.0f + tt);
                    p[e] = s * tt;
                }
                const bool full = (c0 + 32 <= wb.lim_min) && !(wb.any_hole && c0 + 32 > hist_k && c0 < wb.hole_hi_max);
                if (!full) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const int kk = c0 + 16 * (e / 4) + (e % 4);  // + 4 g is folded into the *_lane bounds
                        const bool vis = (kk < lim_lane) && !(kk >= hole_lo_lane && kk < hole_hi_lane);
                        p[e] = vis ? p[e] : 0.f;
                    }
                }
                const u32x4_t pb = {pack2<Tag>(p[0], p[1]), pack2<Tag>(p[2], p[3]), pack2<Tag>(p[4], p[5]),
                                    pack2<Tag>(p[6], p[7])};
                // O^T (D dims x 16 rows) += V^T . P^T
#pragma unroll
                for (int mt = 0; mt < MTILES; ++mt) {
                    const uint16_t* const vp = vt + v_lane_off(mt);
                    const u32x2_t lo = lds_read_tr16_b64(vp);
                    const u32x2_t hi = lds_read_tr16_b64(vp + 16 * D);
                    const u32x4_t va = {lo[0], lo[1], hi[0], hi[1]};
                    o_acc[mt] = mfma16<Tag>(va, pb, o_acc[mt]);
                }
            }
            if constexpr (HAS_RAB) {
                // the block of sub-tile t is free: ask for sub-tile t + 2 (every step, so that the count of open
                // requests says the same thing in every wavefront)
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (S & 1) {
                    request_rab(rab_lo1, rab_hi1, rab_rsrc, rab_voff, static_cast<uint32_t>(t + 2) * 64u);
                } else {
                    request_rab(rab_lo0, rab_hi0, rab_rsrc, rab_voff, static_cast<uint32_t>(t + 2) * 64u);
                }
            }
            // sub-tile t + 1 has landed: at most the requests of this step and of the one before are open (mine),
            // then everybody's
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(kWaitTiles);
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
        };

        // ---- key sweep ----
        // Everything asked for so far is in: the Q fragment and sub-tiles 0 to 2, requested back to back, arrive
        // together.  (The count must be zero here: the compiler counts the Q loads but not the tile requests, and
        // with a wait that leaves four open it would take the Q fragment to be in flight still and wait for it,
        // and with it for every tile request, in front of each product of the sweep.)
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt((0 & 15) | (7 << 4) | (15 << 8));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        HSTU_TL(2);
        for (int t = 0; t < n_sub; t += 4) {
            step(ic0_t{}, t);
            if (t + 1 >= n_sub) {
                break;
            }
            step(ic1_t{}, t + 1);
            if (t + 2 >= n_sub) {
                break;
            }
            step(ic2_t{}, t + 2);
            if (t + 3 >= n_sub) {
                break;
            }
            step(ic3_t{}, t + 3);
        }

        if constexpr (HAS_RAB) {
            // the bias requests of the last two steps name registers that must stay theirs until they have landed
            rab_wait<0>(rab_lo0, rab_hi0);
            rab_wait<0>(rab_lo1, rab_hi1);
        }
        HSTU_TL(3);
        // ---- store O: lane (n, g) holds dims 16 mt + 4 g + 0..3 of query row wr0 + n ----
        const float c_out = a.c_out;
        const int n_e = n, g_e = g, lane_e = lane;
        if (a.out_vec_ok != 0) {
            // every wavefront's requests have landed (the last ones, past the end, move nothing, but they name the
            // slots) and everybody is done reading before anybody writes a slot
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
            // the wavefront's 16 rows pass through 4 KiB of LDS of its own (16-byte chunks XOR-ed with the row) and
            // leave 16 bytes per lane, whole lines per instruction
            uint16_t* const slot_of_wave = (wave & 3) == 0 ? s_k0 : ((wave & 3) == 1 ? s_k1 : ((wave & 3) == 2 ? s_k2 : s_k3));
            uint16_t* const stage = slot_of_wave + (wave >> 2) * (16 * D);
#pragma unroll
            for (int mt = 0; mt < MTILES; ++mt) {
                u32x2_t w;
                w[0] = pack2<Tag>(o_acc[mt][0] * c_out, o_acc[mt][1] * c_out);
                w[1] = pack2<Tag>(o_acc[mt][2] * c_out, o_acc[mt][3] * c_out);
                const int chunk = (2 * mt + (g_e >> 1)) ^ n_e;
                *reinterpret_cast<u32x2_t*>(stage + n_e * D + chunk * 8 + 4 * (g_e & 1)) = w;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            constexpr int RPI = 64 / CPR;    // rows per store instruction
            constexpr int kNonTemporal = 2;  // the rows are not read again by this kernel
            const int rr = lane_e / CPR;
            const int cc = lane_e % CPR;
#pragma unroll
            for (int i = 0; i < kShortWaveM / RPI; ++i) {
                const int r = i * RPI + rr;
                const u32x4_t piece = *reinterpret_cast<const u32x4_t*>(stage + r * D + (cc ^ r) * 8);
                const uint32_t off = (cc * 8 < a.d_v) ? static_cast<uint32_t>(wr0 + r) * o_stride + cc * 16u : kOutOfRange;
                __builtin_amdgcn_raw_buffer_store_b128(piece, o_rsrc, static_cast<int>(off), 0, kNonTemporal);
            }
        } else {
            const uint32_t row_off = static_cast<uint32_t>(wr0 + n_e) * o_stride;
#pragma unroll
            for (int mt = 0; mt < MTILES; ++mt) {
                const int d0 = 16 * mt + 4 * g_e;
                const uint32_t off = (d0 < a.d_v) ? row_off + d0 * 2u : kOutOfRange;
                u32x2_t w;
                w[0] = pack2<Tag>(o_acc[mt][0] * c_out, o_acc[mt][1] * c_out);
                w[1] = pack2<Tag>(o_acc[mt][2] * c_out, o_acc[mt][3] * c_out);
                __builtin_amdgcn_raw_buffer_store_b64(w, o_rsrc, static_cast<int>(off), 0, 0);
            }
        }
    }

#ifdef HSTU_TIMELINE
    if (a.counters != nullptr && tid == 0) {
        __builtin_amdgcn_s_waitcnt(0);
        HSTU_TL(4);
        uint64_t* const rec = reinterpret_cast<uint64_t*>(a.counters) + static_cast<uint64_t>(blockIdx.x) * 8;
        for (int i = 0; i < 5; ++i) {
            rec[i] = tl[i];
        }
        uint32_t xcc = 0, hw = 0;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw));
        rec[5] = (static_cast<uint64_t>(xcc) << 32) | hw;
        rec[6] = live ? 1 : 0;
        rec[7] = static_cast<uint64_t>(slot.level) | (static_cast<uint64_t>(slot.pair) << 16);
    }
#endif
    // ---- rows past the last offset belong to no sequence: zero-fill (all workgroups share the job) ----
    {
        const int64_t first_tail = last_offset < 0 ? 0 : (last_offset < a.total_q ? last_offset : a.total_q);
        const int64_t row_elems = static_cast<int64_t>(a.n_heads_q) * a.d_v;
        const int64_t n_tail = (a.total_q - first_tail) * row_elems;
        uint16_t* tail = out16 + first_tail * row_elems;
        for (int64_t e = static_cast<int64_t>(blockIdx.x) * kShortThreads + tid; e < n_tail;
             e += static_cast<int64_t>(gridDim.x) * kShortThreads) {
            tail[e] = 0;
        }
    }
}

}  // namespace hstu
