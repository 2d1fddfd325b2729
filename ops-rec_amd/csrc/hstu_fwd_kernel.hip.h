// HSTU jagged attention forward for gfx950 (MI355X): device code.
//
// One workgroup (4 wavefronts) owns a 128-row query tile of one (sequence, head); each wavefront
// owns 32 of those rows.  The wavefront keeps its Q rows in registers for the whole key sweep,
// K and V tiles are staged in LDS (double-buffered), and
//
//     S^T = K . Q^T                 v_mfma_f32_32x32x16  (A = K tile from LDS, B = Q from registers)
//     P^T = silu(alpha * (S^T + rab^T)) * scale * mask, rounded to the input type
//     O^T += V^T . P^T              v_mfma_f32_32x32x16  (A = V^T via ds_read_b64_tr_b16, B = P^T)
//
// Computing the transposed score means the accumulator layout of S^T (lane = query row, registers
// = 4 consecutive keys) is exactly the B-operand layout the second product needs, so P never
// leaves registers.  There is no row reduction (no softmax), every output row is produced by
// exactly one wavefront and stored once: no atomics, bitwise deterministic.
//
// What this replaces in the reference (Ascend C):
//   ascendc/attention/hstu_v1/hstu_forward_v1/op_kernel/atlas950/hstu_jagged_forward.cpp:36-62      (entry)
//   .../atlas950/hstu_dense_forward_jagged_kernel.h:257-398                                       (tile loop)
//   .../atlas950/hstu_dense_forward_kernel_patten_bsnd.h:412-470, 493-519, 543-562, 591-689       (QK, score, PV, store)
//   .../atlas950/hstu_dense_causal_mask.h:34-261                                                   (tile classes + mask)
//   .../atlas950/hstu_split_core_policy.h:53-236                                                   (work split)
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hstu {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) short short4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

struct bf16_tag {};
struct f16_tag {};

constexpr int kBlockM = 128;  // query rows per workgroup
constexpr int kWaveM = 32;    // query rows per wavefront
constexpr int kThreads = 256;

struct FwdArgs {
    const void* q;
    const void* k;
    const void* v;
    const void* rab;
    const void* mask;
    void* out;
    const void* offs_q;
    const void* offs_k;
    const void* num_ctx;
    const void* num_tgt;
    int64_t total_q;
    int64_t total_k;
    int n_batch;   // n_offsets - 1
    int n_heads_q;
    int n_heads_k;
    int head_ratio;  // n_heads_q / n_heads_k
    int d_qk;        // real head dims (<= the padded template dims)
    int d_v;
    int max_q;
    int max_k;
    int mask_type;
    int target_group;
    int idx64;       // offsets / context / target are int64
    int n_qtiles;    // ceil(max_q / kBlockM)
    int bh;          // n_batch * n_heads_q
    int rab_vec_ok;  // rab / mask rows may be read 4 elements (8 bytes) at a time
    float c_exp;     // -alpha * log2(e)
    float c_out;     // alpha * silu_scale
};

__device__ __forceinline__ int64_t load_index(const void* p, int64_t i, int idx64)
{
    return idx64 ? static_cast<const int64_t*>(p)[i] : static_cast<int64_t>(static_cast<const int32_t*>(p)[i]);
}

// ---- type helpers -------------------------------------------------------------------------

template <typename Tag>
__device__ __forceinline__ f32x16_t mfma32(u32x4_t a, u32x4_t b, f32x16_t c);

template <>
__device__ __forceinline__ f32x16_t mfma32<bf16_tag>(u32x4_t a, u32x4_t b, f32x16_t c)
{
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                   0, 0, 0);
}
template <>
__device__ __forceinline__ f32x16_t mfma32<f16_tag>(u32x4_t a, u32x4_t b, f32x16_t c)
{
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0,
                                                  0, 0);
}

template <typename Tag>
__device__ __forceinline__ uint32_t pack2(float lo, float hi);  // round-to-nearest-even, lo in bits 0..15
template <>
__device__ __forceinline__ uint32_t pack2<bf16_tag>(float lo, float hi)
{
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
    bf16x2_t r;
    r[0] = static_cast<__bf16>(lo);
    r[1] = static_cast<__bf16>(hi);
    return __builtin_bit_cast(uint32_t, r);
}
template <>
__device__ __forceinline__ uint32_t pack2<f16_tag>(float lo, float hi)
{
    typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
    f16x2_t r;
    r[0] = static_cast<_Float16>(lo);
    r[1] = static_cast<_Float16>(hi);
    return __builtin_bit_cast(uint32_t, r);
}

template <typename Tag>
__device__ __forceinline__ float to_float(uint16_t bits);
template <>
__device__ __forceinline__ float to_float<bf16_tag>(uint16_t bits)
{
    return __builtin_bit_cast(float, static_cast<uint32_t>(bits) << 16);
}
template <>
__device__ __forceinline__ float to_float<f16_tag>(uint16_t bits)
{
    return static_cast<float>(__builtin_bit_cast(_Float16, bits));
}

// ---- LDS layout ---------------------------------------------------------------------------
// K tile: [rows][D] elements, 16-byte chunks XOR-swizzled by row so that the 32x32x16 A-operand
// read (32 lanes = 32 consecutive rows, same logical chunk) spreads over the banks.
template <int D>
__device__ __forceinline__ int k_chunk_swizzle(int row, int chunk)
{
    constexpr int CPR = D / 8;  // 16-byte chunks per row
    if constexpr (CPR >= 16) {
        return chunk ^ (row & 15);
    } else {
        constexpr int RPG = 16 / CPR;  // rows per 256 bytes
        return chunk ^ ((row / RPG) & (CPR - 1));
    }
}
// V tile: [rows][D] elements; the transposed read touches 4 consecutive rows x 64 bytes per
// half-wave, so 64-byte groups are XOR-swizzled by row.
template <int D>
__device__ __forceinline__ int v_chunk_swizzle(int row, int chunk)
{
    constexpr int G = D / 32;  // 64-byte groups per row
    if constexpr (G >= 4) {
        return chunk ^ ((row & 3) << 2);
    } else if constexpr (G == 2) {
        return chunk ^ (((row >> 1) & 1) << 2);
    } else {
        return chunk;
    }
}

__device__ __forceinline__ u32x2_t lds_read_tr16_b64(const uint16_t* p)
{
    typedef short4_t __attribute__((address_space(3))) * lds_ptr_t;
    short4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(p));
    return __builtin_bit_cast(u32x2_t, r);
}

// ---- the kernel ---------------------------------------------------------------------------
// Tag      : bf16_tag / f16_tag
// D        : padded head dim used for both QK and V (32, 64, 128 or 256); real dims come from args
// BN       : keys per LDS tile (multiple of 32)
// HAS_RAB  : attn_bias present
template <typename Tag, int D, int BN, bool HAS_RAB, int MIN_WAVES>
__global__ __launch_bounds__(kThreads, MIN_WAVES) void hstu_fwd_kernel(const FwdArgs a)
{
    constexpr int CPR = D / 8;                        // 16-byte chunks per row
    constexpr int TILE_CHUNKS = BN * CPR;             // chunks per K (or V) tile
    constexpr int LD_PER_THREAD = TILE_CHUNKS / kThreads;
    static_assert(TILE_CHUNKS % kThreads == 0, "tile must split evenly over the workgroup");
    constexpr int KSTEPS = D / 16;   // MFMA steps over the head dim (QK product)
    constexpr int MTILES = D / 32;   // 32-wide output tiles over the head dim (PV product)
    constexpr int NSUB = BN / 32;    // 32-key sub-tiles per LDS tile

    __shared__ __attribute__((aligned(16))) uint16_t s_k[2][BN * D];
    __shared__ __attribute__((aligned(16))) uint16_t s_v[2][BN * D];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int ln = lane & 31;
    const int lh = lane >> 5;

    // ---- which (q-tile, sequence, head): heaviest q-tiles are dispatched first ----
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
    // defensive clamps: malformed offsets must not turn into out-of-bounds addresses
    q1 = q1 < a.total_q ? q1 : a.total_q;
    k1 = k1 < a.total_k ? k1 : a.total_k;
    q0 = q0 < 0 ? 0 : q0;
    k0 = k0 < 0 ? 0 : k0;
    int sq = static_cast<int>(q1 > q0 ? q1 - q0 : 0);
    int sk = static_cast<int>(k1 > k0 ? k1 - k0 : 0);
    sq = sq < a.max_q ? sq : a.max_q;
    sk = sk < a.max_k ? sk : a.max_k;

    uint16_t* const out16 = static_cast<uint16_t*>(a.out);

    // rows past the last offset belong to no sequence: the lightest level zero-fills them
    if (qt == 0) {
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
    const bool wave_active = wr0 < sq;  // inactive wavefronts still help with loads and barriers

    int n_ctx = 0;
    int n_tgt = 0;
    if (a.mask_type == 0) {
        if (a.num_ctx) {
            n_ctx = static_cast<int>(load_index(a.num_ctx, b, a.idx64));
        }
        if (a.num_tgt) {
            n_tgt = static_cast<int>(load_index(a.num_tgt, b, a.idx64));
        }
        n_ctx = n_ctx < 0 ? 0 : n_ctx;
        n_tgt = n_tgt < 0 ? 0 : (n_tgt > sk ? sk : n_tgt);
    }
    const int delta = sk - sq;
    const int hist_k = sk - n_tgt;  // keys before the target block

    // ---- per-row visibility constants (row = this lane's query row, clamped into the sequence) ----
    //   visible(j) = j < lim  &&  !(hole_lo <= j < hole_hi)
    int row = wr0 + ln;
    const bool row_valid = row < sq;
    {
        const int last_row = sq - 1;
        row = row < last_row ? row : last_row;
    }
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
    // wavefront-uniform bounds for tile classification
    int lim_min = lim;
    int lim_max = lim;
    int hole_hi_max = hole_hi;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const int o_min = __shfl_xor(lim_min, off);
        const int o_max = __shfl_xor(lim_max, off);
        const int o_hh = __shfl_xor(hole_hi_max, off);
        lim_min = o_min < lim_min ? o_min : lim_min;
        lim_max = o_max > lim_max ? o_max : lim_max;
        hole_hi_max = o_hh > hole_hi_max ? o_hh : hole_hi_max;
    }
    const bool any_hole = hole_hi_max > hist_k && n_tgt > 0 && a.target_group > 0;

    // ---- keys needed by this workgroup ----
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
    const int n_kt = (kmax + BN - 1) / BN;

    // ---- Q fragment: lane (ln, lh) holds Q[row][16*js + 8*lh .. +7] for js = 0..KSTEPS-1 ----
    u32x4_t qf[KSTEPS];
    {
        const uint16_t* qrow = static_cast<const uint16_t*>(a.q) +
                               ((q0 + wr0 + ln) * a.n_heads_q + h) * static_cast<int64_t>(a.d_qk);
#pragma unroll
        for (int js = 0; js < KSTEPS; ++js) {
            const int d0 = 16 * js + 8 * lh;
            u32x4_t val = {0u, 0u, 0u, 0u};
            if (row_valid && d0 < a.d_qk) {
                val = *reinterpret_cast<const u32x4_t*>(qrow + d0);
            }
            qf[js] = val;
        }
    }

    f32x16_t o_acc[MTILES];
#pragma unroll
    for (int mt = 0; mt < MTILES; ++mt) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            o_acc[mt][i] = 0.f;
        }
    }

    // ---- K/V tile movement: global -> registers -> LDS ----
    const uint16_t* const kbase = static_cast<const uint16_t*>(a.k);
    const uint16_t* const vbase = static_cast<const uint16_t*>(a.v);
    const int64_t k_row_stride = static_cast<int64_t>(a.n_heads_k) * a.d_qk;
    const int64_t v_row_stride = static_cast<int64_t>(a.n_heads_k) * a.d_v;
    u32x4_t k_stage[LD_PER_THREAD];
    u32x4_t v_stage[LD_PER_THREAD];

    auto load_tile = [&](int kt) {
#pragma unroll
        for (int i = 0; i < LD_PER_THREAD; ++i) {
            const int idx = tid + i * kThreads;
            const int r = idx / CPR;
            const int c = idx - r * CPR;
            const int key = kt * BN + r;
            u32x4_t kv = {0u, 0u, 0u, 0u};
            u32x4_t vv = {0u, 0u, 0u, 0u};
            if (key < sk) {
                if (c * 8 < a.d_qk) {
                    kv = *reinterpret_cast<const u32x4_t*>(kbase + (k0 + key) * k_row_stride +
                                                           static_cast<int64_t>(hk) * a.d_qk + c * 8);
                }
                if (c * 8 < a.d_v) {
                    vv = *reinterpret_cast<const u32x4_t*>(vbase + (k0 + key) * v_row_stride +
                                                           static_cast<int64_t>(hk) * a.d_v + c * 8);
                }
            }
            k_stage[i] = kv;
            v_stage[i] = vv;
        }
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int i = 0; i < LD_PER_THREAD; ++i) {
            const int idx = tid + i * kThreads;
            const int r = idx / CPR;
            const int c = idx - r * CPR;
            *reinterpret_cast<u32x4_t*>(&s_k[buf][r * D + k_chunk_swizzle<D>(r, c) * 8]) = k_stage[i];
            *reinterpret_cast<u32x4_t*>(&s_v[buf][r * D + v_chunk_swizzle<D>(r, c) * 8]) = v_stage[i];
        }
    };

    const uint16_t* const rab16 = static_cast<const uint16_t*>(a.rab);
    const uint16_t* const mask16 = static_cast<const uint16_t*>(a.mask);
    const int64_t bias_row =
        ((static_cast<int64_t>(b) * a.n_heads_q + h) * a.max_q + (wr0 + ln)) * static_cast<int64_t>(a.max_k);
    const bool use_custom_mask = (a.mask_type == 3);

    if (n_kt > 0) {
        load_tile(0);
        store_tile(0);
    }
    __syncthreads();

    for (int kt = 0; kt < n_kt; ++kt) {
        const int buf = kt & 1;
        const bool has_next = kt + 1 < n_kt;
        if (has_next) {
            load_tile(kt + 1);
        }

        if (wave_active) {
#pragma unroll
            for (int ms = 0; ms < NSUB; ++ms) {
                const int c0 = kt * BN + ms * 32;  // first key of this 32-key sub-tile
                if (c0 >= lim_max) {
                    continue;  // no row of this wavefront sees any of these keys
                }
                // ---- S^T = K . Q^T (+ rab^T) ----
                f32x16_t s_acc;
                if constexpr (HAS_RAB) {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int j = c0 + 8 * g + 4 * lh;
                        float b0 = 0.f, b1 = 0.f, b2 = 0.f, b3 = 0.f;
                        if (row_valid) {
                            const uint16_t* p = rab16 + bias_row + j;
                            if (a.rab_vec_ok && j + 3 < sk) {
                                const u32x2_t w = *reinterpret_cast<const u32x2_t*>(p);
                                b0 = to_float<Tag>(static_cast<uint16_t>(w[0] & 0xffffu));
                                b1 = to_float<Tag>(static_cast<uint16_t>(w[0] >> 16));
                                b2 = to_float<Tag>(static_cast<uint16_t>(w[1] & 0xffffu));
                                b3 = to_float<Tag>(static_cast<uint16_t>(w[1] >> 16));
                            } else {
                                if (j + 0 < sk) b0 = to_float<Tag>(p[0]);
                                if (j + 1 < sk) b1 = to_float<Tag>(p[1]);
                                if (j + 2 < sk) b2 = to_float<Tag>(p[2]);
                                if (j + 3 < sk) b3 = to_float<Tag>(p[3]);
                            }
                        }
                        s_acc[4 * g + 0] = b0;
                        s_acc[4 * g + 1] = b1;
                        s_acc[4 * g + 2] = b2;
                        s_acc[4 * g + 3] = b3;
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        s_acc[i] = 0.f;
                    }
                }
                {
                    const int kr = ms * 32 + ln;
                    const uint16_t* krow = &s_k[buf][kr * D];
#pragma unroll
                    for (int js = 0; js < KSTEPS; ++js) {
                        const u32x4_t ka =
                            *reinterpret_cast<const u32x4_t*>(krow + k_chunk_swizzle<D>(kr, 2 * js + lh) * 8);
                        s_acc = mfma32<Tag>(ka, qf[js], s_acc);
                    }
                }
                // ---- P^T = silu(alpha * S^T) * scale, masked, rounded to the input type ----
                const bool full = (c0 + 32 <= lim_min) && !(any_hole && c0 + 32 > hist_k && c0 < hole_hi_max) &&
                                  !use_custom_mask;
                uint32_t pk[8];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    float p[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float s = s_acc[4 * g + e];
                        const float ex = __builtin_amdgcn_exp2f(s * a.c_exp);
                        p[e] = (s * a.c_out) * __builtin_amdgcn_rcpf(1.0f + ex);
                    }
                    if (!full) {
                        const int j = c0 + 8 * g + 4 * lh;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int jj = j + e;
                            const bool vis = (jj < lim) && !(jj >= hole_lo && jj < hole_hi);
                            p[e] = vis ? p[e] : 0.f;
                        }
                        if (use_custom_mask) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const int jj = j + e;
                                float m = 0.f;
                                if (row_valid && jj < sk) {
                                    m = to_float<Tag>(mask16[bias_row + jj]);
                                }
                                p[e] *= m;
                            }
                        }
                    }
                    pk[2 * g + 0] = pack2<Tag>(p[0], p[1]);
                    pk[2 * g + 1] = pack2<Tag>(p[2], p[3]);
                }
                // ---- O^T += V^T . P^T ----
#pragma unroll
                for (int j2 = 0; j2 < 2; ++j2) {
                    const u32x4_t pb = {pk[4 * j2 + 0], pk[4 * j2 + 1], pk[4 * j2 + 2], pk[4 * j2 + 3]};
                    const int vr = ms * 32 + 16 * j2 + 4 * lh + ((lane & 15) >> 2);
#pragma unroll
                    for (int mt = 0; mt < MTILES; ++mt) {
                        const int col = 32 * mt + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
                        const int ch = col >> 3;
                        const int within = col & 7;
                        const u32x2_t lo = lds_read_tr16_b64(
                            &s_v[buf][vr * D + v_chunk_swizzle<D>(vr, ch) * 8 + within]);
                        const u32x2_t hi = lds_read_tr16_b64(
                            &s_v[buf][(vr + 8) * D + v_chunk_swizzle<D>(vr + 8, ch) * 8 + within]);
                        const u32x4_t va = {lo[0], lo[1], hi[0], hi[1]};
                        o_acc[mt] = mfma32<Tag>(va, pb, o_acc[mt]);
                    }
                }
            }
        }

        if (has_next) {
            store_tile(buf ^ 1);
        }
        __syncthreads();
    }

    // ---- store O: lane holds query row (wr0 + ln), dims 32*mt + 8*g + 4*lh + 0..3 ----
    if (row_valid) {
        uint16_t* orow = out16 + ((q0 + wr0 + ln) * a.n_heads_q + h) * static_cast<int64_t>(a.d_v);
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d0 = 32 * mt + 8 * g + 4 * lh;
                if (d0 < a.d_v) {
                    u32x2_t w;
                    w[0] = pack2<Tag>(o_acc[mt][4 * g + 0], o_acc[mt][4 * g + 1]);
                    w[1] = pack2<Tag>(o_acc[mt][4 * g + 2], o_acc[mt][4 * g + 3]);
                    *reinterpret_cast<u32x2_t*>(orow + d0) = w;
                }
            }
        }
    }
}

}  // namespace hstu
