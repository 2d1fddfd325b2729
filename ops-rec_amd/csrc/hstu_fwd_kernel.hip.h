// HSTU jagged attention forward for gfx950 (MI355X): device code.
//
// Work item = one 128-row query tile of one (sequence, head): four wavefronts of 32 query rows each.
// The kernel is persistent: a fixed number of workgroups (fwd_wgs_per_cu: two per CU at head dim 128)
// is launched, each builds the work list in its own LDS from seq_offset (sequences bucketed by
// their number of query tiles, heaviest tiles first, tiles past the end of a sequence never
// listed) and then takes item after item: by a fixed schedule over the list (plain variant: no
// device counters at all) or from counters in the caller's workspace (per-XCD queues, split items,
// paged keys), so that the jagged, causal mix of long and short items is balanced and the launch /
// set-up cost of a workgroup is paid once, not per tile.
//
// Per wavefront: its Q rows stay in registers for the whole key sweep of an item; K and V are
// streamed global -> LDS, 32 keys at a time, by buffer loads that write LDS directly (no register
// staging) into two four-slot rings, and
//
//     S^T = K . Q^T                 v_mfma_f32_32x32x16  (A = K sub-tile from LDS, B = Q from registers)
//     P^T = silu(alpha * (S^T + rab^T)) * mask, rounded to the input type
//     O^T += V^T . P^T              v_mfma_f32_32x32x16  (A = V^T via ds_read_b64_tr_b16, B = P^T)
//     O    = (alpha * silu_scale) * O^T^T, rounded once on store
//
// run as a three-deep rolling pipeline (QK of the next sub-tile, SiLU of the current one, PV of the
// previous one in the same time step), so that the matrix pipe and the vector ALU work side by side.
//
// Computing the transposed score means the accumulator layout of S^T (lane = query row, registers
// = 4 consecutive keys) is exactly the B-operand layout the second product needs, so P never
// leaves registers.  There is no row reduction (no softmax), every output row is produced by
// one wavefront and stored once: no atomics on data, bitwise deterministic whatever workgroup
// happens to run an item (split items add their parts in part order).
//
// fp8-e4m3 inputs run the same structure on v_mfma_f32_32x32x64_f8f6f4, with PV contracting over pairs
// of sub-tiles (see "fp8 inputs" at the kernel).
//
// Out-of-range rows (past the end of a sequence) are never branched on: all global accesses go
// through buffer descriptors sized to the sequence, whose out-of-range reads return zero and
// whose out-of-range writes are dropped.
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

#include <type_traits>

#include "hstu_args.h"

namespace hstu {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) short short4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

struct bf16_tag {};
struct f16_tag {};
struct f8_tag {};  // OCP e4m3fn inputs; P is re-quantised to e4m3, the products run on the fp8 MFMA

template <typename Tag>
struct elem_traits {
    static constexpr int kBytes = 2;
    static constexpr bool kF8 = false;
};
template <>
struct elem_traits<f8_tag> {
    static constexpr int kBytes = 1;
    static constexpr bool kF8 = true;
};

constexpr uint32_t kBufferFlags = 0x00020000u;  // raw buffer, 32-bit data format (gfx9 family)
constexpr uint32_t kOutOfRange = 0x80000000u;   // byte offset no descriptor here can contain


__device__ __forceinline__ int64_t load_index(const void* p, int64_t i, int idx64)
{
    return idx64 ? static_cast<const int64_t*>(p)[i] : static_cast<int64_t>(static_cast<const int32_t*>(p)[i]);
}

__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, static_cast<int>(bytes), kBufferFlags);
}

// Visibility bounds shared by the `rows` (32, or 16 in the kernel for short lists) query rows [wr0, min(wr0 + rows, sq)) of one wavefront under the
// built-in mask, in closed form (no cross-lane traffic).  A key j is visible to row i iff
//   j < lim(i)  &&  !(hist_k <= j < hole_hi(i))
// with lim(i) = clamp(i < n_ctx ? max(i + delta + 1, hist_k) : i + delta + 1, 0, sk), delta = sk - sq,
// hist_k = sk - n_tgt, and hole_hi(i) = hist_k + ((i - (sq - n_tgt)) / g) * g for target rows
// (.../op_kernel/atlas950/hstu_dense_causal_mask.h:186-260).  A 32-key tile starting at c0 is
//   skipped    when c0 >= lim_max,
//   unmasked   when c0 + 32 <= lim_min and it does not touch [hist_k, hole_hi_max).
struct WaveBounds {
    int lim_min;
    int lim_max;
    int hole_hi_max;
    bool any_hole;
};

__device__ __forceinline__ WaveBounds wave_bounds(int mask_type, int wr0, int sq, int sk, int n_ctx, int n_tgt,
                                                  int group, bool active, int rows = kWaveM)
{
    WaveBounds w;
    w.hole_hi_max = 0;
    w.any_hole = false;
    if (!active) {
        w.lim_min = 0;
        w.lim_max = 0;
        return w;
    }
    if (mask_type != 0) {
        w.lim_min = sk;
        w.lim_max = sk;
        return w;
    }
    const int wr1 = (wr0 + rows < sq) ? wr0 + rows : sq;
    const int delta = sk - sq;
    const int hist_k = sk - n_tgt;
    int hi = wr1 + delta;  // lim of the last row
    if (wr0 < n_ctx) {
        hi = hi > hist_k ? hi : hist_k;
    }
    int lo = 0x7fffffff;
    if (wr0 < n_ctx) {  // first context row
        const int c = wr0 + delta + 1;
        lo = c > hist_k ? c : hist_k;
    }
    const int rn = wr0 > n_ctx ? wr0 : n_ctx;  // first row that is not a context row
    if (rn < wr1) {
        const int c = rn + delta + 1;
        lo = c < lo ? c : lo;
    }
    w.lim_max = hi < 0 ? 0 : (hi > sk ? sk : hi);
    w.lim_min = lo < 0 ? 0 : (lo > sk ? sk : lo);
    if (n_tgt > 0 && group > 0) {
        const int ti = (wr1 - 1) - (sq - n_tgt);
        if (ti >= 0) {
            w.hole_hi_max = hist_k + (ti / group) * group;
            w.any_hole = w.hole_hi_max > hist_k;
        }
    }
    return w;
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

// fp8: D[32][32] += A[32][64] . B[64][32] on e4m3 operands, v_mfma_f32_32x32x64_f8f6f4 (both formats fp8, no block scales):
// twice the rate per product term of the 32x32x16 form.  Lane (i, half) holds the 32 consecutive k values
// 32 * half .. + 31 of row i of A (column i of B), lowest k in the lowest byte of the first register (checked on
// the device against a host product); the accumulator layout is that of every 32x32 MFMA.
typedef __attribute__((ext_vector_type(8))) int i32x8_t;
__device__ __forceinline__ f32x16_t mfma32x64_f8(u32x4_t a_lo, u32x4_t a_hi, u32x4_t b_lo, u32x4_t b_hi, f32x16_t c)
{
    const i32x8_t a = {static_cast<int>(a_lo[0]), static_cast<int>(a_lo[1]), static_cast<int>(a_lo[2]), static_cast<int>(a_lo[3]),
                       static_cast<int>(a_hi[0]), static_cast<int>(a_hi[1]), static_cast<int>(a_hi[2]), static_cast<int>(a_hi[3])};
    const i32x8_t b = {static_cast<int>(b_lo[0]), static_cast<int>(b_lo[1]), static_cast<int>(b_lo[2]), static_cast<int>(b_lo[3]),
                       static_cast<int>(b_hi[0]), static_cast<int>(b_hi[1]), static_cast<int>(b_hi[2]), static_cast<int>(b_hi[3])};
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}
// two floats -> two e4m3 bytes in the low (hi = false) or high half of `old`; round to nearest even.
// By default the conversion turns magnitudes above 464 into NaN; the fp8 kernels run with the overflow-clamp bit of
// the wavefront's MODE register set (fp8_saturating_conversions()), under which they become +-448 instead (checked
// on the device: 1000 -> 0x7e, -1e30 -> 0xfe), so no clamp is spent per element.
template <bool HI>
__device__ __forceinline__ uint32_t pack2_f8(float a, float b, uint32_t old)
{
    return static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(a, b, static_cast<int>(old), HI));
}

// MODE.FP16_OVFL (bit 23 of hardware register 1): conversions to fp8 (and to fp16) saturate at the largest finite
// value instead of overflowing.  Per wavefront, set once at kernel entry; the state ends with the wavefront.
__device__ __forceinline__ void fp8_saturating_conversions()
{
    __builtin_amdgcn_s_setreg(1 | (23 << 6) | (0 << 11), 1);
}

template <typename Tag>
__device__ __forceinline__ float lo_to_float(uint32_t packed);  // element in bits 0..15
template <typename Tag>
__device__ __forceinline__ float hi_to_float(uint32_t packed);  // element in bits 16..31
template <>
__device__ __forceinline__ float lo_to_float<bf16_tag>(uint32_t packed)
{
    return __builtin_bit_cast(float, packed << 16);
}
template <>
__device__ __forceinline__ float hi_to_float<bf16_tag>(uint32_t packed)
{
    return __builtin_bit_cast(float, packed & 0xffff0000u);
}
template <>
__device__ __forceinline__ float lo_to_float<f16_tag>(uint32_t packed)
{
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(packed & 0xffffu)));
}
template <>
__device__ __forceinline__ float hi_to_float<f16_tag>(uint32_t packed)
{
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(packed >> 16)));
}

// ---- LDS layout ---------------------------------------------------------------------------
// K tile: [rows][D] elements, 16-byte chunks XOR-swizzled by row so that the 32x32x16 A-operand
// read (32 lanes = 32 consecutive rows, same logical chunk) spreads over the banks.
// fp8 tiles (rows of CPR 16-byte chunks), one layout for K and V.  Two read patterns must both be free of
// bank conflicts: the K operand read (16 consecutive rows, one chunk) and the 8-bit transposed V read
// (rows {0,1,2,3,8,9,10,11} + 4 * half, two neighbouring chunks).  The XOR term is therefore a bijection
// of the row bits above the rows-per-256-bytes bits in which row bit 2 (the k-half of the transposed read,
// constant within one of its groups) is moved to the lowest place, so that the other bits separate chunk pairs.
template <int CPR>
__device__ __forceinline__ int chunk_swizzle(int row, int chunk)
{
    if constexpr (CPR >= 16) {
        return chunk ^ ((((row >> 3) & 1) << 3) | (((row >> 1) & 1) << 2) | ((row & 1) << 1) | ((row >> 2) & 1));
    } else if constexpr (CPR == 8) {
        return chunk ^ ((((row >> 3) & 1) << 2) | (((row >> 1) & 1) << 1) | ((row >> 2) & 1));
    } else {
        constexpr int RPG = 16 / CPR;  // rows per 256 bytes
        return chunk ^ ((row / RPG) & (CPR - 1));
    }
}
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

// 8-bit transposed read.  In each group of 16 lanes, lane s supplies the address of 8 bytes M[s][0..7];
// lane i < 8 receives M[0][i], M[2][i], ..., M[14][i] and lane 8 + i receives M[1][i], M[3][i], ..., M[15][i].
__device__ __forceinline__ u32x2_t lds_read_tr8_b64(const uint8_t* p)
{
    typedef __attribute__((ext_vector_type(2))) int i32x2_t;
    typedef i32x2_t __attribute__((address_space(3))) * lds_ptr_t;
    i32x2_t r = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_ptr_t)(p));
    return __builtin_bit_cast(u32x2_t, r);
}

__device__ __forceinline__ u32x2_t lds_read_tr16_b64(const uint16_t* p)
{
    typedef short4_t __attribute__((address_space(3))) * lds_ptr_t;
    short4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(p));
    return __builtin_bit_cast(u32x2_t, r);
}

__device__ __forceinline__ void load_to_lds_b128(__amdgpu_buffer_rsrc_t rsrc, uint16_t* lds_wave_base, uint32_t voffset)
{
    // each lane's 16 bytes land at lds_wave_base + lane * 16; out-of-range sources write zeros
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)lds_wave_base, 16,
                                             static_cast<int>(voffset), 0, 0, 0);
}

// ---- device-side work counters ---------------------------------------------------------------
// The variants that pull items from counters (per-XCD queues, split items, paged keys) keep them in a block at the
// head of the caller's workspace (FwdArgs::counters, kCounterBlockBytes): one work counter per queue, each in a
// 128-byte line of its own, then one arrival counter per split item.  The host clears the block on the launch
// stream ahead of every launch, so the library holds no device state of its own: launches that overlap on one
// GPU, on streams or as replays of captured graphs, are independent as long as their workspaces are.
constexpr int kQueues = 8;          // one work queue per XCD (MI355X: 8 XCDs; workgroup w runs on XCD w mod 8)
constexpr int kCounterStride = 32;  // counters of different queues sit in different 128-byte lines
constexpr int kMaxSplitItems = 2048;
constexpr int kMaxParts = 8;
constexpr int kSplitCounterBase = kQueues * kCounterStride;  // first arrival counter, in 32-bit words
static_assert((kSplitCounterBase + kMaxSplitItems) * 4 <= kCounterBlockBytes, "the counter block holds all counters");

constexpr int kInteriorMinSteps = 20;  // sweeps shorter than this take the general time step throughout
constexpr int kMaxBatchSlots = 2048;  // sequences per call (the reference's limit)
constexpr int kMaxLevels = 160;       // ceil(20480 / 128) query-tile levels

// scalar (uniform-address) load of an offset / count
__device__ __forceinline__ int64_t load_index_uniform(const void* p, int64_t i, int idx64)
{
    typedef const __attribute__((address_space(4))) int64_t* cptr64_t;
    typedef const __attribute__((address_space(4))) int32_t* cptr32_t;
    if (idx64) {
        return ((cptr64_t)(reinterpret_cast<uintptr_t>(p)))[i];
    }
    return static_cast<int64_t>(((cptr32_t)(reinterpret_cast<uintptr_t>(p)))[i]);
}

// floor(x / d) for 0 <= x < 2^23 and d >= 1, without the long integer-division sequence: the product with the
// hardware reciprocal (accurate to one unit in the last place) is off by less than one, so the truncated
// quotient is off by at most one either way.
__device__ __forceinline__ int div_small(int x, int d)
{
    int q = static_cast<int>(static_cast<float>(x) * __builtin_amdgcn_rcpf(static_cast<float>(d)));
    const int r = x - q * d;
    q += (r >= d) ? 1 : 0;
    q -= (r < 0) ? 1 : 0;
    return q;
}

struct U32Pair {
    uint32_t v[2];
};
struct U32Quad {
    uint32_t v[4];
};

// ---- the kernel ---------------------------------------------------------------------------
// Tag      : bf16_tag / f16_tag
// D        : padded head dim used for both QK and V (32, 64, 128 or 256); real dims come from args
// HAS_RAB  : attn_bias present
// HAS_MASK : mask_type 3 (dense custom mask multiplied in)
//
// Key sweep of one item.  Keys are taken 32 at a time ("sub-tile" x = 0, 1, ...); K and V sub-tiles live
// in two rings of four LDS slots each (sub-tile x in slot x mod 4).  One wavefront runs a three-deep
// rolling pipeline: at time t it issues, interleaved instruction by instruction,
//
//     QK(t+1)   S^T(t+1) = K(t+1) . Q^T            MFMA, accumulates in one register block
//     silu(t)   P^T(t)   = silu(S^T(t)) * mask     VALU + transcendental unit
//     PV(t-1)   O^T     += V^T(t-1) . P^T(t-1)     MFMA, different accumulators
//
// so that neither the matrix pipe nor the vector ALU waits for the other and the two MFMA streams are
// never back-to-back dependent.  Register blocks for S and P alternate with the parity of the sub-tile;
// the loop over t is unrolled four times so that LDS slots and register blocks are compile-time.
//
// Ring protocol (all wavefronts of the workgroup, whether or not their rows need the sub-tile):
//   start of time t : K slot of K(t) and V slot of V(t-2) are free -> request K(t+4) and V(t+2)
//                     (requests past the last sub-tile are sent with an out-of-range offset: they move
//                     no data but keep the number of requests per time step constant)
//   end of time t   : wait until the requests made at time t-2 have landed (they are needed at t+1):
//                     at most the requests of times t-1 and t may be outstanding; then one barrier.
//
// fp8 inputs (Tag = f8_tag; OutTag picks the 16-bit output type): same structure with one-byte elements.  The
// score is brought to its real scale (alpha x per-head dequantisation scales) before SiLU, P^T is clamped to
// +-448 and re-quantised to e4m3 (round to nearest even) before or after silu_scale is applied (fp8_scaled_p), the
// V scale (and silu_scale in the first case) goes on the fp32 output.  Both products run on the 64-deep MFMA
// (v_mfma_f32_32x32x64_f8f6f4, twice the rate of the 16-deep fp8 form): an operand is 32 bytes per lane.  For QK
// these are two 16-byte reads of a K row (and the matching two pieces of the Q fragment: k index (half, byte) =
// dim 16 (2p + half) + byte of piece p); PV contracts over the 64 keys of a pair of sub-tiles, its V^T operand
// being four 8-bit transposed reads (16 keys x 32 dims each) in the order in which P^T holds the keys.  rab and the
// custom mask are e4m3 tensors like q (the plain list and the per-XCD queues; items are not split).
//
// QUEUES: build the per-XCD queue machinery (see "Work queues" below).  It pays on long, jagged batches with many
// items per workgroup; its code is on the path of every item, so launches that cannot profit (the host decides by
// an upper bound on the number of items) use the variant without it.
//
// SPLIT: a list with fewer items than workgroups leaves compute units idle while its longest item runs.  This
// variant cuts the key range of the long items into up to kMaxParts parts that are separate entries of the work
// list ("Splitting long items" below); the host uses it when the list is short and a workspace is supplied.  It
// excludes QUEUES.
//
// PAGED: K / V rows come from a paged cache plus the tail of the k / v inputs (see "Paged keys" below); built on top
// of the SPLIT variant, because its callers (inference: few query rows against a long cache) have short lists.
template <typename Tag, typename OutTag, int D, bool HAS_RAB, bool HAS_MASK, bool QUEUES = false, bool SPLIT = false,
          bool PAGED = false>
__global__ __launch_bounds__(256, fwd_wgs_per_cu(D, HAS_RAB, HAS_MASK)) void hstu_fwd_kernel(const FwdArgs a)
{
    constexpr int kThreads = 256;
    constexpr bool F8 = elem_traits<Tag>::kF8;
    if constexpr (F8) {
        fp8_saturating_conversions();  // P^T beyond +-448 becomes +-448, not NaN (an fp16 output saturates likewise)
    }
    constexpr uint32_t ES = elem_traits<Tag>::kBytes;  // bytes per input element
    static_assert(!F8 || !(HAS_RAB || HAS_MASK) || !SPLIT, "fp8 with rab / custom mask: whole items only");
    static_assert(!F8 || D >= 64, "fp8 rows are at least 64 bytes");
    static_assert(!(QUEUES && SPLIT), "one list policy per variant");
    static_assert(!PAGED || (SPLIT && !F8), "the paged variant builds on the split variant, 16-bit inputs");
    constexpr int CPR = D * ES / 16;             // 16-byte chunks per row
    constexpr int EPC16 = 16 / ES;               // elements per 16-byte chunk
    constexpr int SUB_ELEMS = 32 * D * ES / 2;   // one 32-key sub-tile, in 16-bit units
    constexpr int SUB_KIB = 32 * D * ES / 1024;  // 1 KiB load instructions per sub-tile
    constexpr int LPW = SUB_KIB >= 4 ? SUB_KIB / 4 : 1;  // ... per loading wavefront
    constexpr int NLW = SUB_KIB >= 4 ? 4 : SUB_KIB;      // wavefronts that take part in filling a sub-tile
    constexpr int KSTEPS = D / 16;               // MFMA steps over the head dim (QK product)
    constexpr int MTILES = D / 32;               // 32-wide output tiles over the head dim (PV product)
    constexpr int NCH = KSTEPS;                  // chunks per time step: one QK MFMA + one PV MFMA each
    static_assert(2 * MTILES == NCH, "QK and PV products must have the same number of MFMAs");
    constexpr int VM_OUTSTANDING = 2 * 2 * LPW;  // tile requests of two time steps
    constexpr int kWaitTiles = (VM_OUTSTANDING & 15) | (7 << 4) | (15 << 8) | ((VM_OUTSTANDING >> 4) << 14);
    // fp8: both products on the 64-deep MFMA.  QK takes D / 64 of them per sub-tile; PV contracts over the 64 keys of
    // a PAIR of sub-tiles (2u, 2u + 1), half of its D / 32 output tiles in time step 2u + 2 and half in 2u + 3, so a
    // step carries D / 64 MFMAs of either product.  V sub-tiles are requested two at a time in the even steps.
    constexpr bool K64 = F8;
    constexpr int NCH2 = D / 64;
    constexpr int kWaitEven64 = ((4 * LPW) & 15) | (7 << 4) | (15 << 8);  // after an even step: V, V, K of it and K of the step before
    constexpr int kWaitOdd64 = ((2 * LPW) & 15) | (7 << 4) | (15 << 8);   // after an odd step: its K and the K of the step before
    constexpr uint32_t kPastEnd = 0x40000000u;   // added to a source offset: leaves every descriptor

    // eight separate arrays (not one block) so that the compiler can tell the slot being filled by the
    // asynchronous loads from the slot being read, and does not wait for the loads early
    __shared__ __attribute__((aligned(1024))) uint16_t s_k0[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_k1[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_k2[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_k3[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v0[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v1[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v2[SUB_ELEMS];
    __shared__ __attribute__((aligned(1024))) uint16_t s_v3[SUB_ELEMS];
    // work list
    __shared__ uint8_t s_ntiles[kMaxBatchSlots];          // query tiles of each sequence
    __shared__ uint16_t s_order[kMaxBatchSlots];          // sequences, most query tiles first
    __shared__ uint32_t s_bucket[kMaxLevels + 2];         // histogram, then scatter cursors
    __shared__ uint32_t s_rank_start[kMaxLevels + 2];     // [nt]: number of sequences with more than nt query tiles
    __shared__ uint32_t s_queue_start[QUEUES ? kQueues : 1][kMaxLevels + 2];  // per queue: first item of each level / bucket
    __shared__ uint32_t s_item[12];  // [0..3]: the item handed to the workgroup (valid, query tile, sequence, head); [4]: queue order
                                     // [7]: part | parts << 8, [8]: arrival counter, [9]: first partial buffer, [10]: arrivals before
    // plain list: the next item of the workgroup, decoded one item ahead ([parity][valid, query tile, sequence, head,
    // K/V head, q0 lo/hi, q1 lo/hi, k0 lo/hi, k1 lo/hi, context count, target count])
    __shared__ uint32_t s_next[(!QUEUES && !SPLIT) ? 2 : 1][16];
    __shared__ uint8_t s_parts[SPLIT ? kMaxLevels + 2 : 1];         // parts per item of each level
    __shared__ uint32_t s_split_first[SPLIT ? kMaxLevels + 2 : 1];  // first arrival counter of each split level
    __shared__ uint32_t s_ws_first[SPLIT ? kMaxLevels + 2 : 1];     // first partial buffer of each split level

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = uniform(tid >> 6);
    const int ln = lane & 31;
    const int lh = lane >> 5;

    uint16_t* const out16 = static_cast<uint16_t*>(a.out);
    const int n_levels = a.n_qtiles;
    const int n_heads = a.n_heads_q;
    // Lists by tile: level l holds query tile n_levels - 1 - l (longest sweeps first).  With context rows under the
    // built-in mask the first tile of a sequence sweeps all of its history keys, so it is the longest item of all and
    // goes first: level 0 = tile 0, level l >= 1 = tile n_levels - l.
    const bool ctx_first = a.mask_type == 0 && a.num_ctx != nullptr;
    auto tile_of_level = [&](int l) -> int { return ctx_first ? (l == 0 ? 0 : n_levels - l) : n_levels - 1 - l; };

    // rows past the last offset belong to no sequence and are zero-filled when the workgroup leaves (all workgroups
    // share the job); the offset is requested here, so that nothing waits for it
    const int64_t last_offset = load_index_uniform(a.offs_q, a.n_batch, a.idx64);

    // ---- work list: bucket the sequences by their number of query tiles ----
    for (int i = tid; i <= n_levels; i += kThreads) {
        s_bucket[i] = 0;
    }
    __syncthreads();
    for (int b = tid; b < a.n_batch; b += kThreads) {
        int64_t q0 = load_index(a.offs_q, b, a.idx64);
        int64_t q1 = load_index(a.offs_q, b + 1, a.idx64);
        q1 = q1 < a.total_q ? q1 : a.total_q;
        q0 = q0 < 0 ? 0 : q0;
        int sq = static_cast<int>(q1 > q0 ? q1 - q0 : 0);
        sq = sq < a.max_q ? sq : a.max_q;
        const int nt = (sq + kBlockM - 1) / kBlockM;  // 0 .. n_levels
        s_ntiles[b] = static_cast<uint8_t>(nt);
        atomicAdd(&s_bucket[nt], 1u);
    }
    __syncthreads();
    // Bucket starts in "most tiles first" order: s_rank_start[nt] = number of sequences with more than nt tiles.
    // Thread nt sums the counts above its own level by itself: its reads are independent, so they stream through
    // the LDS back to back, where a prefix walk by one thread waits a full LDS round trip per level (with at most
    // 161 levels the extra additions cost nothing).  In the same pass it gets the first item of list level l = nt
    // of the plain list (one queue, by tile, nothing split): level l' holds the items of query tile
    // n_levels - 1 - l', i.e. n_heads per sequence with more tiles than that, so the levels before l hold
    // n_heads * sum over nt' of count[nt'] * max(0, nt' - (n_levels - l)) items.  (With tile 0 in level 0, level
    // l >= 1 starts after all sequences that have a tile at all plus what stood before level l - 1.)
    static_assert(kMaxLevels + 2 <= kThreads, "one thread per level");
    {
        uint32_t above = 0;
        uint32_t items_before = 0;
        if (tid <= n_levels) {
            const int floor_tiles = n_levels - tid + (ctx_first ? 1 : 0);
            uint32_t with_tiles = 0;
            for (int nt = n_levels; nt >= 1; --nt) {
                const uint32_t c = s_bucket[nt];
                above += nt > tid ? c : 0u;
                with_tiles += c;
                items_before += nt > floor_tiles ? c * static_cast<uint32_t>(nt - floor_tiles) : 0u;
            }
            if (ctx_first) {
                items_before = tid == 0 ? 0u : items_before + with_tiles;
            }
        }
        __syncthreads();  // the counts have been read by everybody
        if (tid <= n_levels) {
            s_rank_start[tid] = above;
            s_bucket[tid] = above;  // from here on: scatter cursors
            if constexpr (!QUEUES && !SPLIT) {
                s_queue_start[0][tid] = items_before * static_cast<uint32_t>(n_heads);
            }
        }
        if constexpr (!QUEUES && !SPLIT) {
            if (tid == 0) {
                s_item[4] = 0u;  // by tile
            }
        }
    }
    __syncthreads();
    // Work queues.  A "pair" is one (sequence, K/V head): its K / V rows are read by every query tile of every
    // query head that shares the K/V head.  Pairs are numbered p = sorted position * n_heads_k + kv head; pair p
    // belongs to queue p mod 8, and a queue is served first by the workgroups of one XCD, so that the rows of a
    // pair are fetched into one L2 instead of eight.  Two orders inside a queue:
    //   by tile  - the heaviest (highest) query tile of all its pairs first, then the next tile down, ...: longest
    //              items first.  With a handful of items per workgroup and item lengths between 1 and
    //              max_seq_len / 32 steps this is what keeps the end of the launch short.  Level l of the queue =
    //              query tile tile_of_level(l) of its pairs that have it (the sequences at sorted positions
    //              [0, s_rank_start[qt]) have more than qt tiles).
    //   by pair  - pair after pair (most tiles first), the tiles of a pair together, heaviest first: the
    //              workgroups of the XCD sweep the K / V rows of few pairs at a time, and each row is fetched
    //              from HBM about once instead of once per query tile.  Bucket l of the queue = its pairs with
    //              nt = n_levels - l tiles (sorted positions [s_rank_start[nt], s_rank_start[nt - 1])).
    // "By pair" starts the heavy tiles of late pairs late; that is harmless when there are many items per
    // workgroup and the late pairs are short (a jagged batch), and costly when all sequences are equally long.
    // It is chosen when the list has at least 4 items per workgroup and the mean tile count of the sequences is
    // at most 0.7 of the largest, and whatever the lengths from 6 items per workgroup on: by tile, the resident workgroups
    // of a long list all work on different pairs, and every item streams its keys from memory (128 x 4 heads of 7621
    // rows, d 128: 61 GB in 11.05 ms by tile, 7.21 ms by pair; 64 x 4 of 4096 rows 1.39 -> 1.14 ms; level at 8 items per
    // workgroup of 1024 or 512 rows).
    // "By tile" runs as ONE queue shared by all workgroups (the order that matters there is global), "by pair" as
    // one queue per XCD.
    if ((QUEUES || SPLIT) && tid < (QUEUES ? kQueues : 1)) {
        bool by_pair = false;
        if constexpr (QUEUES) {
            // total tiles = sum over nt of nt * (sequences with nt tiles); sequences with nt tiles =
            // s_rank_start[nt-1] - s_rank_start[nt]  (every builder thread works the order out for itself)
            uint32_t tiles = 0, seqs = 0;
            int nt_max = 0;
            for (int nt = 1; nt <= n_levels; ++nt) {
                const uint32_t c = s_rank_start[nt - 1] - s_rank_start[nt];
                tiles += c * static_cast<uint32_t>(nt);
                seqs += c;
                nt_max = c != 0 ? nt : nt_max;
            }
            const uint32_t items = tiles * static_cast<uint32_t>(n_heads);
            by_pair = (items >= 4u * gridDim.x && 10u * tiles <= 7u * seqs * static_cast<uint32_t>(nt_max)) || items >= 6u * gridDim.x;
        }
        if (tid == 0) {
            s_item[4] = by_pair ? 1u : 0u;
        }
        const int ratio = a.head_ratio;
        const int n_heads_k = a.n_heads_k;
        // Splitting long items.  Level l holds the items of query tile qt = tile_of_level(l); under the built-in
        // mask such an item sweeps about 4 (qt + 1) sub-tiles (tile 0 with context rows: all), otherwise all of
        // max_seq_len_k.  With `target` = the
        // mean number of time steps per workgroup (3 steps of start-up per item included, never below 8), the items
        // of a level whose nominal length exceeds it are listed as m = ceil(nominal / target) entries (at most
        // kMaxParts), one per part of the key range, next to each other in the list.  Part i sweeps the sub-tiles
        // [i * len, (i + 1) * len) of the item's real range, len a multiple of 4; it writes its fp32 accumulators
        // to its own buffer in the workspace and counts itself in; the part that finds all others counted in adds
        // the m buffers in part order (so the sum does not depend on who came last) and stores the rows.
        // A level is split only while arrival counters and workspace buffers last, and nothing is split when the
        // list has an item for every workgroup anyway: measured on MI355X, an entry of the list costs 4 - 6 us on
        // top of its sweep (its own start-up, the hand-over of its accumulators), which a list of 1.4 items per
        // workgroup (batch 32 x 4 heads, lengths 256..1024) no longer earns back, while a list that leaves workgroups
        // idle (one 20480-row sequence, or 4 sequences x 2 heads up to 3000 rows) finishes in 0.5 - 0.65 of the time.
        // For the same reason the target is raised until the list with its parts still has at most one entry per
        // workgroup: a second round of entries costs more than shorter parts gain (12 x 4 items of 1024 rows:
        // 42.5 us with the mean as the target, 35.2 us with this rule, 33.5 us unsplit).
        uint32_t split_target = 0;
        uint32_t split_items = 0, split_bufs = 0;
        auto nominal_steps = [&](int qt) -> uint32_t {
            const int all = (a.max_k + 31) / 32;
            if (a.mask_type != 0 || (ctx_first && qt == 0)) {
                return static_cast<uint32_t>(all);
            }
            const int causal = 4 * (qt + 1) + (a.max_k > a.max_q ? (a.max_k - a.max_q) / 32 : 0);
            return static_cast<uint32_t>(causal < all ? causal : all);
        };
        if constexpr (SPLIT) {
            uint32_t steps = 0, items = 0;
            for (int l = 0; l < n_levels; ++l) {
                const uint32_t cnt = s_rank_start[tile_of_level(l)] * static_cast<uint32_t>(n_heads);
                steps += cnt * (nominal_steps(tile_of_level(l)) + 3u);
                items += cnt;
            }
            split_target = steps / gridDim.x;
            split_target = split_target < 8u ? 8u : split_target;
            if (a.ws == nullptr || items >= gridDim.x) {
                split_target = 0x7fffffffu;  // nothing is split
            } else {
                // one round: if the list cut at the mean has more entries than there are workgroups, the target
                // is raised so that the entries splitting adds (at most nominal / target per item) go to the
                // workgroups that would have had no item
                // (counted in floating point: one thread does this for up to 160 levels, and the count only picks
                // the rule, so a part more or less at an exact multiple does not matter)
                uint32_t entries = 0;
                const float inv_target = 1.0f / static_cast<float>(split_target);
                for (int l = 0; l < n_levels; ++l) {
                    const uint32_t cnt = s_rank_start[tile_of_level(l)] * static_cast<uint32_t>(n_heads);
                    const uint32_t m = static_cast<uint32_t>(static_cast<float>(nominal_steps(tile_of_level(l))) * inv_target + 0.999f);
                    entries += cnt * (m > static_cast<uint32_t>(kMaxParts) ? static_cast<uint32_t>(kMaxParts) : (m < 1u ? 1u : m));
                }
                if (entries > gridDim.x) {
                    const uint32_t spare = gridDim.x - items;
                    const uint32_t fit = (steps - 3u * items + spare - 1u) / spare;
                    split_target = split_target < fit ? fit : split_target;
                }
            }
        }
        uint32_t acc = 0;
        for (int l = 0; l < n_levels; ++l) {
            s_queue_start[tid][l] = acc;
            if constexpr (SPLIT) {
                const uint32_t cnt = s_rank_start[tile_of_level(l)] * static_cast<uint32_t>(n_heads);
                uint32_t m = (nominal_steps(tile_of_level(l)) + split_target - 1u) / split_target;
                m = m > static_cast<uint32_t>(kMaxParts) ? static_cast<uint32_t>(kMaxParts) : m;
                if (m > 1u && (split_items + cnt > static_cast<uint32_t>(kMaxSplitItems) || split_bufs + cnt * m > a.ws_parts)) {
                    m = 1u;
                }
                s_parts[l] = static_cast<uint8_t>(m);
                s_split_first[l] = split_items;
                s_ws_first[l] = split_bufs;
                if (m > 1u) {
                    split_items += cnt;
                    split_bufs += cnt * m;
                }
                acc += cnt * m;
                continue;
            }
            if (by_pair) {
                const int nt = n_levels - l;
                const uint32_t p0 = s_rank_start[nt] * static_cast<uint32_t>(n_heads_k);
                const uint32_t p1 = s_rank_start[nt - 1] * static_cast<uint32_t>(n_heads_k);
                // pairs p in [p0, p1) with p mod 8 == tid
                const uint32_t mine = (p1 + kQueues - 1 - tid) / kQueues - (p0 + kQueues - 1 - tid) / kQueues;
                acc += mine * static_cast<uint32_t>(nt * ratio);
            } else if (tid == 0) {
                acc += s_rank_start[tile_of_level(l)] * static_cast<uint32_t>(n_heads);  // every pair that has this tile
            }
        }
        s_queue_start[tid][n_levels] = acc;
    }
    __syncthreads();
    // Stable scatter (sequences of one bucket stay in index order) by wavefront 0 alone: every workgroup
    // must arrive at the very same list, which an order-of-arrival scatter over four wavefronts would
    // not give.  64 sequences per trip; lanes holding the same tile count are ranked with a ballot.
    // (the cursors of all 64 sequences of a trip are read in one go before the loop over the distinct tile counts
    // among them, which then runs on ballots alone: no LDS round trip per distinct count)
    if (wave == 0) {
        for (int base = 0; base < a.n_batch; base += 64) {
            const int b = base + lane;
            const bool valid = b < a.n_batch;
            const int key = valid ? static_cast<int>(s_ntiles[valid ? b : 0]) : -1;
            const uint32_t start = s_bucket[valid ? key : 0];
            uint32_t before = 0;
            uint64_t todo = __builtin_amdgcn_ballot_w64(valid);
            while (todo != 0) {
                const int leader = __builtin_ctzll(todo);
                const int k0 = __builtin_amdgcn_readlane(key, leader);
                const bool mine = valid && key == k0;
                const uint64_t same = __builtin_amdgcn_ballot_w64(mine);
                if (mine) {
                    before = __builtin_popcountll(same & ((1ull << lane) - 1ull));
                }
                if (lane == leader) {
                    s_bucket[k0] = start + static_cast<uint32_t>(__builtin_popcountll(same));
                }
                todo &= ~same;
            }
            if (valid) {
                s_order[start + before] = static_cast<uint16_t>(b);
            }
        }
    }
    __syncthreads();

    // ---- per-lane constants that do not depend on the item ----
    const uint32_t q_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_qk * ES;  // bytes per row
    const uint32_t k_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_qk * ES;
    const uint32_t v_stride = static_cast<uint32_t>(a.n_heads_k) * a.d_v * ES;
    const uint32_t o_stride = static_cast<uint32_t>(a.n_heads_q) * a.d_v * 2u;  // the output is 16-bit
    // K / V sub-tile streaming: load instruction i of this wavefront fills LDS bytes
    // [(wave * LPW + i) * 1024, +1024) of a slot; per-lane source offsets are fixed, only the base moves
    uint32_t k_src[LPW];
    uint32_t v_src[LPW];
    int ld_row[LPW];  // row of the sub-tile that load i of this lane fills (paged variant)
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
        const int slot = (wave * LPW + i) * 64 + lane;  // 16-byte slot within the sub-tile
        const int r = (slot / CPR) & 31;
        ld_row[i] = r;
        const int pc = slot % CPR;
        const int kc = F8 ? chunk_swizzle<CPR>(r, pc) : k_chunk_swizzle<D>(r, pc);  // XOR swizzles are their own inverse
        const int vc = F8 ? chunk_swizzle<CPR>(r, pc) : v_chunk_swizzle<D>(r, pc);
        k_src[i] = (kc * EPC16 < a.d_qk) ? static_cast<uint32_t>(r) * k_stride + kc * 16u : kOutOfRange;
        v_src[i] = (vc * EPC16 < a.d_v) ? static_cast<uint32_t>(r) * v_stride + vc * 16u : kOutOfRange;
    }
    // LDS read offsets relative to a sub-tile (16-bit inputs: in elements; fp8: in bytes)
    constexpr int KREADS = F8 ? KSTEPS / 2 : KSTEPS;  // fp8: one 16-byte read feeds two MFMA steps
    int k_lane_off[KREADS];
    int v_lane_off[MTILES];
    if constexpr (F8) {
#pragma unroll
        for (int jp = 0; jp < KREADS; ++jp) {
            k_lane_off[jp] = ln * D + chunk_swizzle<CPR>(ln, 2 * jp + lh) * 16;
        }
        // transposed read of 16 keys x 32 dims: source lane s of a 16-lane group g supplies 8 dims of one key,
        //   key  = 8 * ((s / 2) / 4) + 4 * (g / 2) + (s / 2) % 4   (so that byte j of k-half g / 2 is the key P^T holds there)
        //   dims = 32 * mt + 16 * (g % 2) + 8 * (s % 2) .. + 7
        const int s16 = lane & 15;
        const int g16 = lane >> 4;
        const int key = 8 * ((s16 >> 1) >> 2) + 4 * (g16 >> 1) + ((s16 >> 1) & 3);
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
            const int col = 32 * mt + 16 * (g16 & 1) + 8 * (s16 & 1);
            v_lane_off[mt] = key * D + chunk_swizzle<CPR>(key, col >> 4) * 16 + (col & 15);
        }
    } else {
#pragma unroll
        for (int js = 0; js < KREADS; ++js) {
            k_lane_off[js] = ln * D + k_chunk_swizzle<D>(ln, 2 * js + lh) * 8;
        }
        const int vr0 = 4 * lh + ((lane & 15) >> 2);
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
            const int col = 32 * mt + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
            v_lane_off[mt] = vr0 * D + v_chunk_swizzle<D>(vr0, col >> 3) * 8 + (col & 7);
        }
    }
    float c_exp = a.c_exp;
    float c_out = a.c_out;
    float c_x = 1.0f;  // fp8 only: raw score -> alpha * (dequantised score)
    float c_p = 1.0f;  // fp8 only: what P is multiplied by before it is quantised (1, or silu_scale)
    float c_pi = 1.0f;  // fp8 only: 1 / c_p, and 1 / (c_x c_p): the factors of (1 + t) in the sigmoid's reciprocal
    float c_qi = 1.0f;
    // rab is added to S^T by the matrix pipe: S^T += E_j . R_j (j = 0, 1), where R_j holds, per lane (query row,
    // half lh), the 8 consecutive rab values of keys 16 lh + 8 j .. + 7 exactly as they lie in memory (B operand)
    // and E_j is the constant 0/1 matrix that routes k-slot (lh, e) to key row 16 lh + 8 j + e (A operand).
    // This costs two MFMAs per sub-tile and no conversion, lane exchange or add on the vector ALU.
    u32x4_t rab_route[2] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
    if constexpr (HAS_RAB) {
        const uint32_t one = std::is_same<Tag, bf16_tag>::value ? 0x3f80u : 0x3c00u;  // 1.0 in the input type
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int d = ln - 16 * lh - 8 * j;  // the element of this lane's row that is 1, if in 0..7
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                rab_route[j][i] = (d == 2 * i) ? one : (d == 2 * i + 1) ? (one << 16) : 0u;
            }
        }
    }
    const int bias_mode = a.bias_vec_ok;  // 0: element loads, 1: 8-byte loads, 2: 16-byte loads + lane exchange

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

    // =============================== item loop ===============================
    // The first item of a workgroup is fixed (workgroup w: item w / nq of queue w mod nq, nq = number of queues);
    // later ones are pulled from the queue's counter.  With the pull, the position of the next non-empty queue is
    // read as well: a workgroup whose queue is drained moves on to that queue if it still has items (and so on
    // around the ring), otherwise it leaves.  Every queue keeps the workgroups of its own XCD until it is empty,
    // so moving on only ever adds help.  One lane does this bookkeeping and the decoding of the item and hands
    // the result to the workgroup through LDS.
    // (run by wavefront 0 as a whole, with uniform control flow: the levels of the list are searched by its lanes
    // side by side, one ballot per 64 levels, where a walk by one thread waits an LDS round trip per level; the
    // counters are touched by lane 0 alone)
    int fq_queue = 0;           // the queue this workgroup pulls from
    uint32_t fq_idx = 0;        // the item index it holds in that queue
    bool fq_first = true;       // nothing pulled yet
    auto fetch_item = [&]() {   // executed by wavefront 0
        const bool by_pair = QUEUES && s_item[4] != 0;
        const int nq = by_pair ? kQueues : 1;
        const int nq_shift = by_pair ? 3 : 0;
        const int ratio = a.head_ratio;
        const int n_heads_k = a.n_heads_k;
        unsigned int* const counters = a.counters;
        auto fixed_items = [&](int qu) -> uint32_t {  // workgroups qu, qu + nq, ... took the first items of queue qu
            return gridDim.x > static_cast<uint32_t>(qu) ? (gridDim.x - qu + nq - 1) >> nq_shift : 0u;
        };
        auto next_queue = [&](int qu) -> int {  // the next queue after qu that has items at all (qu itself if there is none)
            for (int i = 1; i < nq; ++i) {
                const int cand = (qu + i) & (nq - 1);
                if (s_queue_start[cand][n_levels] != 0) {
                    return cand;
                }
            }
            return qu;
        };
        // pulls the next index of queue qu and, when `peek` names another queue, reads where that one stands
        auto pull = [&](int qu, int peek, uint32_t& peeked) -> uint32_t {
            uint32_t got = 0, seen = 0;
            if (lane == 0) {
                got = atomicAdd(&counters[qu * kCounterStride], 1u);
                if (peek != qu) {
                    seen = __hip_atomic_load(&counters[peek * kCounterStride], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            peeked = static_cast<uint32_t>(uniform(static_cast<int>(seen)));
            return static_cast<uint32_t>(uniform(static_cast<int>(got)));
        };
        auto no_item = [&]() {
            if (lane == 0) {
                s_item[0] = 0;
            }
        };
        uint32_t other_next = 0;  // where the next non-empty queue stands, as far as known
        bool other_known = false;
        if (fq_first) {
            fq_first = false;
            fq_queue = static_cast<int>(blockIdx.x) & (nq - 1);
            fq_idx = blockIdx.x >> nq_shift;
        } else {
            const int other = next_queue(fq_queue);
            uint32_t seen = 0;
            const uint32_t got = pull(fq_queue, other, seen);
            if (other != fq_queue) {
                other_next = fixed_items(other) + seen;
                other_known = true;
            }
            fq_idx = fixed_items(fq_queue) + got;
        }
        while (fq_idx >= s_queue_start[fq_queue][n_levels]) {
            // this queue is drained (or empty from the start): help the next one if it has work left
            const int other = next_queue(fq_queue);
            if (other == fq_queue) {
                no_item();
                return;
            }
            if (!other_known) {
                other_next = fixed_items(other);  // optimistic: nothing pulled there yet
            }
            if (other_next >= s_queue_start[other][n_levels]) {
                no_item();
                return;
            }
            fq_queue = other;
            const int after = next_queue(other);
            uint32_t seen = 0;
            const uint32_t got = pull(other, after, seen);
            other_known = after != other;
            if (other_known) {
                other_next = fixed_items(after) + seen;
            }
            fq_idx = fixed_items(other) + got;
        }
        // level of the item: the number of levels that end at or before it
        int lvl = 0;
        for (int base = 0; base < n_levels; base += 64) {
            const int l = base + lane;
            const bool ends_before = l < n_levels && s_queue_start[fq_queue][(l < n_levels ? l : 0) + 1] <= fq_idx;
            lvl += __builtin_popcountll(__builtin_amdgcn_ballot_w64(ends_before));
        }
        lvl = lvl < n_levels - 1 ? lvl : n_levels - 1;
        const int j_item = static_cast<int>(fq_idx - s_queue_start[fq_queue][lvl]);
        int qt, p_item, r_item;
        uint32_t part_word = 0, split_counter = 0, split_buffer = 0;
        if (by_pair) {
            // item j of bucket lvl (pairs with nt tiles) = pair j / (nt * ratio) of this queue there, query tile
            // nt - 1 - (j % (nt * ratio)) / ratio, query head (kv head) * ratio + j % ratio
            const int nt_item = n_levels - lvl;
            const int per_pair = nt_item * ratio;
            const int m_item = div_small(j_item, per_pair);
            const int rem_item = j_item - m_item * per_pair;
            const int t_item = div_small(rem_item, ratio);
            qt = nt_item - 1 - t_item;
            if (a.mask_type == 0 && a.num_ctx != nullptr) {
                // with context rows the first tile of a sequence sweeps all of its history keys: it goes ahead of the pair's
                // other tiles instead of last, where it would end the launch with one long item per queue
                qt = t_item == 0 ? 0 : nt_item - t_item;
            }
            r_item = rem_item - t_item * ratio;
            const int p_first = static_cast<int>(s_rank_start[nt_item]) * n_heads_k;
            p_item = p_first + ((fq_queue + kQueues - (p_first & (kQueues - 1))) & (kQueues - 1)) + m_item * kQueues;
        } else {
            // item j of level lvl (query tile qt) = pair j / ratio, query head (kv head) * ratio + j % ratio
            qt = tile_of_level(lvl);
            int j_whole = j_item;
            if constexpr (SPLIT) {
                // entry j of a split level = part j % m of item j / m
                const int m = s_parts[lvl];
                j_whole = div_small(j_item, m);
                part_word = static_cast<uint32_t>(j_item - j_whole * m) | (static_cast<uint32_t>(m) << 8);
                split_counter = s_split_first[lvl] + static_cast<uint32_t>(j_whole);
                split_buffer = s_ws_first[lvl] + static_cast<uint32_t>(j_whole * m);
            }
            p_item = div_small(j_whole, ratio);
            r_item = j_whole - p_item * ratio;
        }
        const int rank = div_small(p_item, n_heads_k);
        const int hk_item = p_item - rank * n_heads_k;
        const uint32_t seq_item = s_order[rank];
        if (lane == 0) {
            s_item[0] = 1;
            s_item[1] = static_cast<uint32_t>(qt);
            s_item[2] = seq_item;
            s_item[3] = static_cast<uint32_t>(hk_item * ratio + r_item);
            s_item[5] = (static_cast<uint32_t>(fq_queue) << 28) | fq_idx;  // (for the development item log)
            s_item[6] = static_cast<uint32_t>(hk_item);
            if constexpr (SPLIT) {
                s_item[7] = part_word;
                s_item[8] = split_counter;
                s_item[9] = split_buffer;
            }
        }
    };
    // Plain list (one queue, by tile, nothing split): no counter at all.  The items of workgroup w are fixed by the
    // list alone: in round r it takes item r * grid + w (r even) or r * grid + grid - 1 - w (r odd), so that the
    // workgroups whose item of one round was heaviest get the lightest of the next -- what pulling from a counter
    // gives such a short list as well (measured equal on MI355X), without the counter's round trip, without device
    // state shared between launches, and with the next item known in advance: wavefront 0 decodes it, offsets
    // included, while the tile requests of the current item are under way, and leaves it in LDS for the others.
    constexpr bool kStaticList = !QUEUES && !SPLIT;
    auto decode_ahead = [&](int round) {  // executed by wavefront 0; fills s_next[round & 1]
        uint32_t(&rec)[16] = s_next[kStaticList ? (round & 1) : 0];
        const uint32_t g = gridDim.x;
        const uint32_t idx = static_cast<uint32_t>(round) * g + ((round & 1) ? g - 1u - blockIdx.x : blockIdx.x);
        if (idx >= s_queue_start[0][n_levels]) {
            if (lane == 0) {
                rec[0] = 0;
            }
            return;
        }
        int lvl = 0;
        for (int base = 0; base < n_levels; base += 64) {
            const int l = base + lane;
            const bool ends_before = l < n_levels && s_queue_start[0][(l < n_levels ? l : 0) + 1] <= idx;
            lvl += __builtin_popcountll(__builtin_amdgcn_ballot_w64(ends_before));
        }
        lvl = lvl < n_levels - 1 ? lvl : n_levels - 1;
        const int j_item = static_cast<int>(idx - s_queue_start[0][lvl]);
        const int p_item = div_small(j_item, a.head_ratio);
        const int r_item = j_item - p_item * a.head_ratio;
        const int rank = div_small(p_item, a.n_heads_k);
        const int hk_item = p_item - rank * a.n_heads_k;
        const int seq = uniform(static_cast<int>(s_order[rank]));
        const int64_t q0 = load_index_uniform(a.offs_q, seq, a.idx64);
        const int64_t q1 = load_index_uniform(a.offs_q, seq + 1, a.idx64);
        const int64_t k0 = load_index_uniform(a.offs_k, seq, a.idx64);
        const int64_t k1 = load_index_uniform(a.offs_k, seq + 1, a.idx64);
        int ctx = 0, tgt = 0;
        if (a.mask_type == 0) {
            if (a.num_ctx) {
                ctx = static_cast<int>(load_index_uniform(a.num_ctx, seq, a.idx64));
            }
            if (a.num_tgt) {
                tgt = static_cast<int>(load_index_uniform(a.num_tgt, seq, a.idx64));
            }
        }
        if (lane == 0) {
            rec[1] = static_cast<uint32_t>(tile_of_level(lvl));
            rec[2] = static_cast<uint32_t>(seq);
            rec[3] = static_cast<uint32_t>(hk_item * a.head_ratio + r_item);
            rec[4] = static_cast<uint32_t>(hk_item);
            rec[5] = static_cast<uint32_t>(q0);
            rec[6] = static_cast<uint32_t>(static_cast<uint64_t>(q0) >> 32);
            rec[7] = static_cast<uint32_t>(q1);
            rec[8] = static_cast<uint32_t>(static_cast<uint64_t>(q1) >> 32);
            rec[9] = static_cast<uint32_t>(k0);
            rec[10] = static_cast<uint32_t>(static_cast<uint64_t>(k0) >> 32);
            rec[11] = static_cast<uint32_t>(k1);
            rec[12] = static_cast<uint32_t>(static_cast<uint64_t>(k1) >> 32);
            rec[13] = static_cast<uint32_t>(ctx);
            rec[14] = static_cast<uint32_t>(tgt);
            rec[0] = 1;
        }
    };
    int round = 0;
    if constexpr (kStaticList) {
        if (wave == 0) {
            decode_ahead(0);
        }
        __syncthreads();
    }
    for (;;) {
        int qt, b, h, hk;
        int64_t q0, q1, k0, k1;
        int n_ctx = 0;
        int n_tgt = 0;
        if constexpr (kStaticList) {
            const uint32_t(&rec)[16] = s_next[kStaticList ? (round & 1) : 0];
            if (rec[0] == 0) {
                break;
            }
            auto word = [&](int i) -> uint32_t { return static_cast<uint32_t>(uniform(static_cast<int>(rec[i]))); };
            qt = static_cast<int>(word(1));
            b = static_cast<int>(word(2));
            h = static_cast<int>(word(3));
            hk = static_cast<int>(word(4));
            q0 = static_cast<int64_t>(word(5) | (static_cast<uint64_t>(word(6)) << 32));
            q1 = static_cast<int64_t>(word(7) | (static_cast<uint64_t>(word(8)) << 32));
            k0 = static_cast<int64_t>(word(9) | (static_cast<uint64_t>(word(10)) << 32));
            k1 = static_cast<int64_t>(word(11) | (static_cast<uint64_t>(word(12)) << 32));
            n_ctx = static_cast<int>(word(13));
            n_tgt = static_cast<int>(word(14));
        } else {
            if (wave == 0) {
                fetch_item();
            }
            __syncthreads();
            if (s_item[0] == 0) {
                break;
            }
            qt = uniform(static_cast<int>(s_item[1]));
            b = uniform(static_cast<int>(s_item[2]));
            h = uniform(static_cast<int>(s_item[3]));
            hk = uniform(static_cast<int>(s_item[6]));
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

        const int r0 = qt * kBlockM;  // < sq by construction of the work list
        const int wr0 = r0 + wave * kWaveM;
        const bool wave_active = wr0 < sq;  // inactive wavefronts still take part in loads and barriers

        if (a.mask_type == 0) {
            n_ctx = n_ctx < 0 ? 0 : n_ctx;
            n_tgt = n_tgt < 0 ? 0 : (n_tgt > sk ? sk : n_tgt);
        }
        const int delta = sk - sq;
        const int hist_k = sk - n_tgt;  // keys before the target block

        // Paged keys.  Key rows [0, n_cached) of the sequence are rows of its pages page_ids[page_first ..
        // page_last), page_size rows each, in order; key rows [n_cached, sk) are the last n_new rows of its segment
        // of the k / v inputs.  page_size is a multiple of 32, so a 32-key sub-tile lies in one page; the sub-tile
        // that holds row n_cached takes its rows from both sources (two requests under complementary lane masks).
        // The physical page of sub-tile x is kept in pid_ring[x mod 4]: it is looked up (a scalar load) one time
        // step before the request for K(x) needs it and stays until the request for V(x), two steps later, is out.
        // (All of this runs on the scalar unit, which the wavefronts of a CU share: the per-step part is kept to a
        // handful of 32-bit instructions; 64-bit products are formed once per item.)
        int n_new = 0, n_cached = 0;
        int page_first = 0, page_hi = 0;  // indices into page_ids: first page of the sequence, last valid index
        int pid_ring[4] = {0, 0, 0, 0};
        const uint8_t* cache_head = nullptr;       // row 0 of page 0, this K/V head
        uint32_t page_bytes = 0;                   // one page of K (or V) rows
        if constexpr (PAGED) {
            if (a.num_tgt) {
                n_new = static_cast<int>(load_index_uniform(a.num_tgt, b, a.idx64));
            }
            n_new = n_new < 0 ? 0 : (n_new > sk ? sk : n_new);
            n_new = n_new > sq ? sq : n_new;
            n_cached = sk - n_new;
            const int64_t pf = load_index_uniform(a.page_offsets, b, a.idx64);
            const int64_t pl = load_index_uniform(a.page_offsets, b + 1, a.idx64);
            const int64_t top = a.n_page_ids - 1;
            const int64_t hi = (pl - 1 < top) ? pl - 1 : top;
            page_hi = static_cast<int>(hi < 0 ? 0 : hi);
            page_first = static_cast<int>(pf < 0 ? 0 : (pf > page_hi ? page_hi : pf));
            cache_head = static_cast<const uint8_t*>(a.kv_cache) + static_cast<int64_t>(hk) * a.d_qk * ES;
            page_bytes = k_stride << a.page_shift;
        }
        const int sub_shift = a.page_shift - 5;  // sub-tiles per page, as a shift
        const int last_pid = static_cast<int>(a.num_pages - 1);
        auto page_of = [&](int x) -> int {
            int idx = page_first + (x >> sub_shift);
            idx = idx < page_hi ? idx : page_hi;
            int pid = static_cast<int>(load_index_uniform(a.page_ids, idx, a.idx64));
            pid = pid < last_pid ? pid : last_pid;
            return pid < 0 ? 0 : pid;
        };

        // ---- buffer descriptors sized to this sequence / head ----
        const __amdgpu_buffer_rsrc_t q_rsrc =
            make_rsrc(static_cast<const uint8_t*>(a.q) + (q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_qk) * ES,
                      static_cast<uint32_t>(sq - 1) * q_stride + a.d_qk * ES);
        // (paged variant: the descriptors of the new rows, i.e. the last n_new rows of the segment of k / v)
        const int64_t k_first_row = PAGED ? q1 - n_new : k0;
        const int k_rows = PAGED ? n_new : sk;
        const __amdgpu_buffer_rsrc_t k_rsrc =
            make_rsrc(static_cast<const uint8_t*>(a.k) + (k_first_row * a.n_heads_k + hk) * static_cast<int64_t>(a.d_qk) * ES,
                      k_rows > 0 ? static_cast<uint32_t>(k_rows - 1) * k_stride + a.d_qk * ES : 0u);
        const __amdgpu_buffer_rsrc_t v_rsrc =
            make_rsrc(static_cast<const uint8_t*>(a.v) + (k_first_row * a.n_heads_k + hk) * static_cast<int64_t>(a.d_v) * ES,
                      k_rows > 0 ? static_cast<uint32_t>(k_rows - 1) * v_stride + a.d_v * ES : 0u);
        const __amdgpu_buffer_rsrc_t o_rsrc =
            make_rsrc(out16 + (q0 * a.n_heads_q + h) * static_cast<int64_t>(a.d_v),
                      static_cast<uint32_t>(sq - 1) * o_stride + a.d_v * 2u);

        if constexpr (F8) {
            // per-head dequantisation scales: score scale alpha * qs * ks, output scale silu_scale * vs
            typedef const __attribute__((address_space(4))) float* cfloat_t;
            const float qs = a.q_descale ? ((cfloat_t)(reinterpret_cast<uintptr_t>(a.q_descale)))[h] : 1.0f;
            const float ks = a.k_descale ? ((cfloat_t)(reinterpret_cast<uintptr_t>(a.k_descale)))[hk] : 1.0f;
            const float vs = a.v_descale ? ((cfloat_t)(reinterpret_cast<uintptr_t>(a.v_descale)))[hk] : 1.0f;
            c_x = a.alpha * qs * ks;
            c_exp = -1.4426950408889634f * c_x;
            // where silu_scale is applied: to the fp32 output (P quantised at its own scale), or, the reference's
            // rounding point, to P before it is quantised (fp8_scaled_p)
            c_out = (a.fp8_scaled_p ? 1.0f : a.silu_scale) * vs;
            c_p = a.fp8_scaled_p ? a.silu_scale : 1.0f;
            c_pi = 1.0f / c_p;
            c_qi = 1.0f / (c_x * c_p);
        }

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
        const int n_sub = (kmax + 31) / 32;  // sub-tiles swept for the item
        // the part of them this entry of the list stands for
        int x_begin = 0;
        int x_end = n_sub;
        int part = 0;
        int n_parts = 1;
        if constexpr (SPLIT) {
            part = uniform(static_cast<int>(s_item[7] & 0xffu));
            n_parts = uniform(static_cast<int>(s_item[7] >> 8));
            if (n_parts > 1) {
                const int len = ((n_sub + n_parts - 1) / n_parts + 3) & ~3;
                x_begin = part * len;
                x_begin = x_begin < n_sub ? x_begin : n_sub;
                x_end = x_begin + len < n_sub ? x_begin + len : n_sub;
            }
        }

        // requests for K sub-tile xk into K slot KS and V sub-tile xv into V slot VS
        // paged variant: sub-tile x of K (kv = 0) or V (kv = 1), physical page pid, into dst.  Rows below `bnd`
        // come from the page, the others from the new rows; a request past the end moves nothing.
        auto request_paged = [&](uint16_t* dst, const __amdgpu_buffer_rsrc_t new_rsrc, const uint32_t (&src)[LPW], int x,
                                 int pid, int kv) {
            const bool live = x < x_end;
            const int bnd = live ? n_cached - x * 32 : 0;
            const int rows_c = bnd < 0 ? 0 : (bnd > 32 ? 32 : bnd);
            const uint32_t in_page = static_cast<uint32_t>(x & ((1 << sub_shift) - 1)) * 32u * k_stride;
            const uint64_t page_off = static_cast<uint64_t>(static_cast<uint32_t>(2 * pid + kv)) * page_bytes + in_page;
            const __amdgpu_buffer_rsrc_t page_rsrc =
                make_rsrc(cache_head + page_off, rows_c > 0 ? static_cast<uint32_t>(rows_c - 1) * k_stride + a.d_qk * ES : 0u);
            // offset of sub-tile row 0 among the new rows (negative, as a wrapped unsigned, while bnd > 0: the
            // lanes that use it have rows >= bnd, which brings the sum back into range)
            const uint32_t new_base = live ? static_cast<uint32_t>(x * 32 - n_cached) * k_stride : kPastEnd;
#pragma unroll
            for (int i = 0; i < LPW; ++i) {
                if (ld_row[i] < bnd) {
                    load_to_lds_b128(page_rsrc, dst + (wave * LPW + i) * 512, src[i]);
                } else {
                    load_to_lds_b128(new_rsrc, dst + (wave * LPW + i) * 512, src[i] + new_base);
                }
            }
        };
        auto request_k = [&](auto ks, int xk) {
            if (NLW == 4 || wave < NLW) {
                uint16_t* const dst = k_slot(ks);
                if constexpr (PAGED) {
                    request_paged(dst, k_rsrc, k_src, xk, pid_ring[decltype(ks)::value & 3], 0);
                } else {
                    const uint32_t kb = (xk < x_end) ? static_cast<uint32_t>(xk * 32) * k_stride : kPastEnd;
#pragma unroll
                    for (int i = 0; i < LPW; ++i) {
                        load_to_lds_b128(k_rsrc, dst + (wave * LPW + i) * 512, k_src[i] + kb);
                    }
                }
            }
        };
        auto request_v = [&](auto vs, int xv) {
            if (NLW == 4 || wave < NLW) {
                uint16_t* const dst = v_slot(vs);
                if constexpr (PAGED) {
                    request_paged(dst, v_rsrc, v_src, xv, pid_ring[decltype(vs)::value & 3], 1);
                } else {
                    const uint32_t vb = (xv < x_end) ? static_cast<uint32_t>(xv * 32) * v_stride : kPastEnd;
#pragma unroll
                    for (int i = 0; i < LPW; ++i) {
                        load_to_lds_b128(v_rsrc, dst + (wave * LPW + i) * 512, v_src[i] + vb);
                    }
                }
            }
        };
        typedef std::integral_constant<int, 0> ic0_t;
        typedef std::integral_constant<int, 1> ic1_t;
        typedef std::integral_constant<int, 2> ic2_t;
        typedef std::integral_constant<int, 3> ic3_t;

        // ---- start-up: what the times before the first would have requested, and the Q fragment ----
        // (x_begin is a multiple of 4: sub-tile x_begin + i belongs in slot i)
        if constexpr (PAGED) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                pid_ring[i] = page_of(x_begin + i);
            }
        }
        request_k(ic0_t{}, x_begin);
        if constexpr (!K64) {
            request_v(ic0_t{}, x_begin);  // (64-deep PV: V(x_begin) and V(x_begin + 1) go out in time step x_begin)
        }
        request_k(ic1_t{}, x_begin + 1);
        request_k(ic2_t{}, x_begin + 2);
        // Q fragment: lane (ln, lh) holds Q[row][16*js + 8*lh .. +7] for js = 0..KSTEPS-1
        // (fp8: 16 bytes per pair of steps, dims 16 * (2 * jp + lh) .. + 15, low half for step 2 jp)
        u32x4_t qf[KREADS];
        {
            const uint32_t row_off = static_cast<uint32_t>(wr0 + ln) * q_stride;
#pragma unroll
            for (int js = 0; js < KREADS; ++js) {
                const int d0 = F8 ? 32 * js + 16 * lh : 16 * js + 8 * lh;
                const uint32_t off = (d0 < a.d_qk) ? row_off + d0 * ES : kOutOfRange;
                qf[js] = __builtin_amdgcn_raw_buffer_load_b128(q_rsrc, static_cast<int>(off), 0, 0);
            }
        }

        // the next item of this workgroup, while the requests of this one are under way
        if constexpr (kStaticList) {
            if (wave == 0) {
                decode_ahead(round + 1);
            }
        }

        // ---- per-row visibility constants (row = this lane's query row, clamped into the sequence) ----
        //   visible(j) = j < lim  &&  !(hole_lo <= j < hole_hi)
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
        const int lim_min = wb.lim_min;
        const int hole_hi_max = wb.hole_hi_max;
        const bool any_hole = wb.any_hole;
        const int nx_all = (wb.lim_max + 31) / 32;  // sub-tiles this wavefront's rows can see (<= n_sub)
        const int nx_w = (SPLIT && x_end < nx_all) ? x_end : nx_all;  // ... and the end of what it works on in this part
        // Context rows: the sub-tiles [rows_only_from, rows_only_to) of this wavefront lie past the limit of every row
        // of its that is not a context row and wholly below the limit of every context row (and before the target keys,
        // when target rows carve holes): a row sees such a sub-tile whole or not at all, and its visibility is one
        // comparison per lane instead of one per score.  These are nearly all steps of a sequence's first query tile.
        int rows_only_from = 0, rows_only_to = 0;
        if (a.mask_type == 0 && wave_active && wr0 < n_ctx) {
            const int wr1 = (wr0 + kWaveM < sq) ? wr0 + kWaveM : sq;
            int other_hi = n_ctx < wr1 ? wr1 + delta : 0;  // limit of the last row that is not a context row
            other_hi = other_hi < 0 ? 0 : (other_hi > sk ? sk : other_hi);
            int ctx_lo = wr0 + delta + 1 > hist_k ? wr0 + delta + 1 : hist_k;  // limit of the first context row
            ctx_lo = (any_hole && ctx_lo > hist_k) ? hist_k : ctx_lo;
            ctx_lo = ctx_lo < 0 ? 0 : (ctx_lo > sk ? sk : ctx_lo);
            rows_only_from = (other_hi + 31) >> 5;
            rows_only_to = ctx_lo >> 5;
        }
        // (one scalar register: the d = 128 variants have none to spare)
        const uint32_t rows_only = static_cast<uint32_t>(uniform(rows_only_from | (rows_only_to << 16)));
        // per-lane bounds relative to the lane's first key of a sub-tile (key = c0 + 4*lh + kk)
        const int lim_lane = lim - 4 * lh;
        const int hole_lo_lane = hole_lo - 4 * lh;
        const int hole_hi_lane = hole_hi - 4 * lh;

        // ---- rab / custom mask: per (sequence, head) descriptor, rows indexed by the local (i, j) ----
        const uint32_t bias_bytes = static_cast<uint32_t>(a.max_q) * static_cast<uint32_t>(a.max_k) * ES;
        const int64_t bias_plane =
            (static_cast<int64_t>(b) * a.n_heads_q + h) * a.max_q * static_cast<int64_t>(a.max_k);
        const __amdgpu_buffer_rsrc_t rab_rsrc =
            make_rsrc(HAS_RAB ? static_cast<const uint8_t*>(a.rab) + bias_plane * ES : nullptr, HAS_RAB ? bias_bytes : 0u);
        const __amdgpu_buffer_rsrc_t mask_rsrc = make_rsrc(
            HAS_MASK ? static_cast<const uint8_t*>(a.mask) + bias_plane * ES : nullptr, HAS_MASK ? bias_bytes : 0u);
        const uint32_t bias_row_off = static_cast<uint32_t>(wr0 + ln) * static_cast<uint32_t>(a.max_k) * ES;

        // fp8 inputs: rab and the custom mask are e4m3 tensors like q.  The 16 values of a 32-key sub-tile a lane
        // needs -- keys c0 + 8 g + 4 lh + 0..3 for g = 0..3, the order of its score registers -- are four words of
        // four bytes (one 32-bit load each when rows are 4-byte aligned, byte loads otherwise); they are turned into
        // floats on the vector ALU where they are used (the reference adds the bias and multiplies the mask in fp32 as
        // well, op_kernel/atlas950/hstu_dense_forward_kernel_patten_bsnd.h:412-470).
        auto load_bias_f8 = [&](__amdgpu_buffer_rsrc_t rsrc, int c0, uint32_t (&w)[8]) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const uint32_t off = bias_row_off + static_cast<uint32_t>(c0 + 8 * g + 4 * lh);
                if (bias_mode != 0) {
                    w[g] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, static_cast<int>(off), 0, 0);
                } else {
                    uint32_t eoff = off;
                    asm volatile("" : "+v"(eoff));
                    uint32_t word = 0;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t byte = __builtin_amdgcn_raw_buffer_load_b8(rsrc, static_cast<int>(eoff + e), 0, 0);
                        word |= (byte & 0xffu) << (8 * e);
                    }
                    w[g] = word;
                }
            }
        };
        // element e (0..15, score register order) of such a block of words, as a float
        auto f8_element = [&](const uint32_t (&w)[8], int e) -> float {
            const uint32_t word = w[e / 4];
            switch (e % 4) {
            case 0:
                return __builtin_amdgcn_cvt_f32_fp8(static_cast<int>(word), 0);
            case 1:
                return __builtin_amdgcn_cvt_f32_fp8(static_cast<int>(word), 1);
            case 2:
                return __builtin_amdgcn_cvt_f32_fp8(static_cast<int>(word), 2);
            default:
                return __builtin_amdgcn_cvt_f32_fp8(static_cast<int>(word), 3);
            }
        };

        // Requests the rab values of keys c0 + 16 lh .. + 15 of this lane's row, 8 packed words in memory order
        // (what the routing MFMAs above take as their B operands).
        auto load_rab = [&](int c0, uint32_t (&w)[8]) {
            const uint32_t off = bias_row_off + static_cast<uint32_t>(c0 + 16 * lh) * 2u;
            if (bias_mode == 2) {
                const U32Quad t0 = __builtin_bit_cast(U32Quad, __builtin_amdgcn_raw_buffer_load_b128(rab_rsrc, static_cast<int>(off), 0, 0));
                const U32Quad t1 = __builtin_bit_cast(U32Quad, __builtin_amdgcn_raw_buffer_load_b128(rab_rsrc, static_cast<int>(off + 16u), 0, 0));
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    w[i] = t0.v[i];
                    w[4 + i] = t1.v[i];
                }
            } else if (bias_mode == 1) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const U32Pair t = __builtin_bit_cast(
                        U32Pair, __builtin_amdgcn_raw_buffer_load_b64(rab_rsrc, static_cast<int>(off + 8u * i), 0, 0));
                    w[2 * i + 0] = t.v[0];
                    w[2 * i + 1] = t.v[1];
                }
            } else {
                uint32_t eoff = off;
                asm volatile("" : "+v"(eoff));  // (keeps the optimiser from relating these to the vector loads above)
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint32_t e0 = __builtin_amdgcn_raw_buffer_load_b16(rab_rsrc, static_cast<int>(eoff + 4u * i), 0, 0);
                    const uint32_t e1 = __builtin_amdgcn_raw_buffer_load_b16(rab_rsrc, static_cast<int>(eoff + 4u * i + 2u), 0, 0);
                    w[i] = (e0 & 0xffffu) | (e1 << 16);
                }
            }
        };
        // Requests the 16 bias (or mask) values of one 32-key sub-tile as 8 packed words; order_bias() must be
        // applied to the words once they are about to be used.
        // Mode 2 (rows 16-byte aligned): the two lanes of a row (lh = 0, 1) read 32 contiguous bytes each (keys
        // 16 lh .. 16 lh + 15), i.e. the row's 64 bytes in two 16-byte loads per lane instead of four 8-byte
        // loads; the accumulator layout wants keys 8g + 4 lh + 0..3 per lane, so the lanes exchange half of
        // what they read (v_permlane32_swap, in order_bias).
        auto load_bias = [&](__amdgpu_buffer_rsrc_t rsrc, int c0, uint32_t (&w)[8]) {
            if (bias_mode == 2) {
                const uint32_t off = bias_row_off + static_cast<uint32_t>(c0 + 16 * lh) * 2u;
                const U32Quad t0 = __builtin_bit_cast(U32Quad, __builtin_amdgcn_raw_buffer_load_b128(rsrc, static_cast<int>(off), 0, 0));
                const U32Quad t1 = __builtin_bit_cast(U32Quad, __builtin_amdgcn_raw_buffer_load_b128(rsrc, static_cast<int>(off + 16u), 0, 0));
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    w[i] = t0.v[i];
                    w[4 + i] = t1.v[i];
                }
                return;
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const uint32_t off = bias_row_off + static_cast<uint32_t>(c0 + 8 * g + 4 * lh) * 2u;
                if (bias_mode == 1) {
                    // (reinterpreted as a struct before its words are taken: taking integer elements
                    // straight from the builtin's vector result is narrowed to a one-element load by the
                    // optimiser of this toolchain)
                    const U32Pair t = __builtin_bit_cast(
                        U32Pair, __builtin_amdgcn_raw_buffer_load_b64(rsrc, static_cast<int>(off), 0, 0));
                    w[2 * g + 0] = t.v[0];
                    w[2 * g + 1] = t.v[1];
                } else {
                    // the offset is laundered through an empty asm so that the optimiser cannot relate
                    // these element loads to the vector load of the other branch
                    uint32_t eoff = off;
                    asm volatile("" : "+v"(eoff));
                    const uint32_t e0 = __builtin_amdgcn_raw_buffer_load_b16(rsrc, static_cast<int>(eoff), 0, 0);
                    const uint32_t e1 = __builtin_amdgcn_raw_buffer_load_b16(rsrc, static_cast<int>(eoff + 2u), 0, 0);
                    const uint32_t e2 = __builtin_amdgcn_raw_buffer_load_b16(rsrc, static_cast<int>(eoff + 4u), 0, 0);
                    const uint32_t e3 = __builtin_amdgcn_raw_buffer_load_b16(rsrc, static_cast<int>(eoff + 6u), 0, 0);
                    w[2 * g + 0] = (e0 & 0xffffu) | (e1 << 16);
                    w[2 * g + 1] = (e2 & 0xffffu) | (e3 << 16);
                }
            }
        };

        // brings requested words into accumulator order (word 2g, 2g+1 = keys 8g + 4 lh + 0..3)
        auto order_bias = [&](uint32_t (&w)[8]) {
            if (bias_mode == 2) {
                // lane (row, 0) holds words d0..d7 (keys 0..15), lane (row, 1) d8..d15; lh = 0 wants d0 d1 d4 d5 d8 d9
                // d12 d13, lh = 1 wants d2 d3 d6 d7 d10 d11 d14 d15: words 2, 3, 6, 7 of the lower half-wave trade
                // places with words 0, 1, 4, 5 of the upper one
                typedef __attribute__((ext_vector_type(2))) unsigned u2_t;
#pragma unroll
                for (int i = 0; i < 2; ++i) {
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const u2_t r = __builtin_amdgcn_permlane32_swap(w[4 * i + j], w[4 * i + 2 + j], false, false);
                        w[4 * i + j] = r[0];
                        w[4 * i + 2 + j] = r[1];
                    }
                }
                // now {w0 w1 | w2 w3 | w4 w5 | w6 w7} = groups g = {0 | 2 | 1 | 3}
                const uint32_t t2 = w[2], t3 = w[3];
                w[2] = w[4];
                w[3] = w[5];
                w[4] = t2;
                w[5] = t3;
            }
        };

        f32x16_t o_acc[MTILES];
#pragma unroll
        for (int mt = 0; mt < MTILES; ++mt) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                o_acc[mt][i] = 0.f;
            }
        }
        // register blocks of the rolling pipeline: sub-tile x uses block x & 1
        f32x16_t s_blk0, s_blk1;     // S^T
        uint32_t p_blk0[8], p_blk1[8];  // P^T, packed pairs
        uint32_t p_blk2[8], p_blk3[8];  // 64-deep PV only: sub-tile x uses P^T block x & 3 (a pair is consumed two and three steps on)
        uint32_t rabw0[8], rabw1[8];  // rab words of sub-tile x in block x & 1
        uint32_t mw0[8], mw1[8];      // custom mask words of sub-tile x in block x & 1
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            s_blk0[i] = 0.f;
            s_blk1[i] = 0.f;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            p_blk0[i] = 0;
            p_blk1[i] = 0;
            p_blk2[i] = 0;
            p_blk3[i] = 0;
            rabw0[i] = 0;
            rabw1[i] = 0;
            mw0[i] = 0;
            mw1[i] = 0;
        }
        if constexpr (HAS_RAB && !F8) {
            if (nx_w > x_begin) {
                load_rab(x_begin * 32, rabw0);
            }
        }

        // one time step, for this wavefront; S = t mod 4.  INTERIOR (compile time) promises that sub-tiles t - 1, t
        // and t + 1 all exist for this wavefront, that sub-tile t is fully visible and (with rab) that sub-tile t + 2
        // exists: the step is then straight-line code -- no flags, no branches, a dozen scalar instructions.
        // (Measured on MI355X: 3 - 6 % on sweeps of 32 steps and more; the general step spends about fifty scalar
        // instructions and ten branches on its flags.)
        auto time_step = [&](auto sc, auto interior, const int t) {
            constexpr int S = decltype(sc)::value;
            constexpr bool INTERIOR = decltype(interior)::value;
            constexpr int PAR = S & 1;  // parity of t
            const f32x16_t& s_cur = PAR ? s_blk1 : s_blk0;  // S^T(t), transformed in this step
            f32x16_t& s_nxt = PAR ? s_blk0 : s_blk1;        // S^T(t+1), accumulated in this step
            // P^T block of sub-tile x: x & 1, or x & 3 with the 64-deep PV
            auto p_block = [&](auto ic) -> uint32_t(&)[8] {
                constexpr int I = decltype(ic)::value & 3;
                if constexpr (I == 0) {
                    return p_blk0;
                } else if constexpr (I == 1) {
                    return p_blk1;
                } else if constexpr (I == 2) {
                    return p_blk2;
                } else {
                    return p_blk3;
                }
            };
            uint32_t(&pk_cur)[8] = p_block(std::integral_constant<int, K64 ? S : PAR>{});        // P^T(t), written
            const uint32_t(&pk_prev)[8] = p_block(std::integral_constant<int, PAR ? 0 : 1>{});   // P^T(t-1), consumed (32-deep PV)
            // 64-deep PV: the pair of sub-tiles consumed in this step, t - 2 and t - 1 (t even) or t - 3 and t - 2 (t odd)
            constexpr int LO = PAR ? (S + 1) & 3 : (S + 2) & 3;
            constexpr int HI = (LO + 1) & 3;
            const int t0 = PAR ? t - 3 : t - 2;
            uint32_t(&mw_cur)[8] = PAR ? mw1 : mw0;               // custom mask words of sub-tile t
            uint32_t(&mw_nxt)[8] = PAR ? mw0 : mw1;
            uint32_t(&rab_far)[8] = PAR ? rabw1 : rabw0;          // receives rab(t+2)
            uint32_t(&rab_nxt)[8] = PAR ? rabw0 : rabw1;          // rab(t+1)
            const uint16_t* const kt = k_slot(std::integral_constant<int, (S + 1) & 3>{});  // K(t+1)
            const uint16_t* const vt = v_slot(std::integral_constant<int, (S + 3) & 3>{});  // V(t-1)
            const int c0 = t * 32;

            const bool do_qk = INTERIOR || t + 1 < nx_w;
            const bool do_silu = INTERIOR || (t >= x_begin && t < nx_w);
            const bool do_pv = INTERIOR || (K64 ? (t0 >= x_begin && t0 < nx_w) : (t >= x_begin + 1 && t <= nx_w));
            const bool full = INTERIOR || ((c0 + 32 <= lim_min) && !(any_hole && c0 + 32 > hist_k && c0 < hole_hi_max));

            // (1) bias / mask requests for later steps; they go out before the tile requests of this step so
            //     that waiting for them never waits for a younger tile
            // (a 16-bit bias is requested between the two MFMA blocks, below: measured a little better than here,
            // C3 61.8 -> 60.6 us, and better than behind the tile requests at the end of the step, 63.4 us)
            if constexpr (HAS_RAB && F8) {
                if (do_qk) {
                    load_bias_f8(rab_rsrc, c0 + 32, rab_nxt);  // used one step on, by the SiLU of sub-tile t + 1
                }
            }
            if constexpr (HAS_MASK) {
                if (do_qk) {
                    if constexpr (F8) {
                        load_bias_f8(mask_rsrc, c0 + 32, mw_nxt);
                    } else {
                        load_bias(mask_rsrc, c0 + 32, mw_nxt);
                    }
                }
            }
            // (2) tile requests of this time step.  With a 16-bit bias they go out at the end of the step, just ahead of
            //     the wait, instead of here behind the bias requests (measured: C3 64.3 -> 62.3 us, C4 407 -> 403 us,
            //     4096-key uniform sequences with bias 447 -> 437 us; without a bias the place makes no difference)
            constexpr bool kRequestsAtEnd = HAS_RAB && !F8;
            auto tile_requests = [&]() {
                if constexpr (K64) {
                    // V(t) and V(t + 1), both in the even steps (their slots held V(t - 4) and V(t - 3), read for the last
                    // time in step t - 1), ahead of K so that the wait after an odd step may leave two K requests open
                    if constexpr (!PAR) {
                        request_v(std::integral_constant<int, S>{}, t);
                        request_v(std::integral_constant<int, (S + 1) & 3>{}, t + 1);
                    }
                    request_k(sc, t + 4);
                } else {
                    request_k(sc, t + 4);
                    request_v(std::integral_constant<int, (S + 2) & 3>{}, t + 2);
                }
                if constexpr (PAGED) {
                    pid_ring[(S + 1) & 3] = page_of(t + 5);  // for the request of K(t + 5) in the next time step
                }
            };
            if constexpr (!kRequestsAtEnd) {
                tile_requests();
            }

            // (3) arithmetic.  Two straight-line blocks, each entered on one wavefront-uniform flag:
            //       block A (sub-tile t-1 exists):  PV(t-1) MFMAs with the first half of silu(t) between them
            //       block B (sub-tile t+1 exists):  QK(t+1) MFMAs with the second half of silu(t) between them
            //     Every accumulator is updated at exactly one place in the code.  Inside a block nothing is
            //     conditional: at the two ends of a sweep the SiLU half of a block may work on a score block
            //     that holds no sub-tile; what it writes is never consumed.  Visibility is applied afterwards,
            //     to the packed P^T, and only in the steps whose sub-tile is not fully visible.
            // K operand read r (16-bit inputs: MFMA step r; fp8: steps 2r and 2r+1) and V^T operand of chunk c
            auto read_k = [&](int r) -> u32x4_t {
                if constexpr (F8) {
                    return *reinterpret_cast<const u32x4_t*>(reinterpret_cast<const uint8_t*>(kt) + k_lane_off[r]);
                } else {
                    return *reinterpret_cast<const u32x4_t*>(kt + k_lane_off[r]);
                }
            };
            // chunk c of the PV block = key half c % 2 of output tile c / 2: two consecutive MFMAs accumulate into the
            // same registers
            auto read_v = [&](int c) -> u32x4_t {
                const int j2 = c % 2, mt = c / 2;
                const uint16_t* p = vt + v_lane_off[mt] + 16 * j2 * D;
                const u32x2_t lo = lds_read_tr16_b64(p);
                const u32x2_t hi = lds_read_tr16_b64(p + 8 * D);
                const u32x4_t r = {lo[0], lo[1], hi[0], hi[1]};
                return r;
            };
            // unmasked P^T pair i (score elements 2i, 2i+1)
            auto silu_pair = [&](int i) {
                float tt[2], p[2];
                if constexpr (F8 && HAS_RAB) {
                    // the score at its real scale with the bias: x = alpha (qs ks S + rab); (rab_far is the block of the
                    // parity of t: it was filled one step ago)
                    float x[2];
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        x[e] = __builtin_fmaf(s_cur[2 * i + e], c_x, a.alpha * f8_element(rab_far, 2 * i + e));
                        tt[e] = __builtin_amdgcn_exp2f(x[e] * -1.4426950408889634f);
                    }
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        // x sigmoid(x) c_p = x / ((1 + t) / c_p)
                        p[e] = x[e] * __builtin_amdgcn_rcpf(__builtin_fmaf(tt[e], c_pi, c_pi));
                    }
                    if constexpr (HAS_MASK) {
                        p[0] *= f8_element(mw_cur, 2 * i);
                        p[1] *= f8_element(mw_cur, 2 * i + 1);
                    }
                    if (i & 1) {
                        pk_cur[i / 2] = pack2_f8<true>(p[0], p[1], pk_cur[i / 2]);
                    } else {
                        pk_cur[i / 2] = pack2_f8<false>(p[0], p[1], pk_cur[i / 2]);
                    }
                    return;
                }
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    tt[e] = s_cur[2 * i + e] * c_exp;
                }
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    tt[e] = __builtin_amdgcn_exp2f(tt[e]);
                }
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    if constexpr (F8) {
                        // the scale that brings P^T to where it is quantised rides on the reciprocal:
                        // s sigma c_q = s / ((1 + t) / c_q)
                        tt[e] = __builtin_fmaf(tt[e], c_qi, c_qi);
                    } else {
                        tt[e] = 1.0f + tt[e];
                    }
                }
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    tt[e] = __builtin_amdgcn_rcpf(tt[e]);
                }
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    p[e] = s_cur[2 * i + e] * tt[e];
                }
                if constexpr (HAS_MASK) {
                    if constexpr (F8) {
                        p[0] *= f8_element(mw_cur, 2 * i);
                        p[1] *= f8_element(mw_cur, 2 * i + 1);
                    } else {
                        p[0] *= lo_to_float<Tag>(mw_cur[i]);
                        p[1] *= hi_to_float<Tag>(mw_cur[i]);
                    }
                }
                if constexpr (F8) {
                    // (P^T is at its real scale, times silu_scale at the reference's rounding point: see c_qi);
                    // pair i = bytes 2 (i % 2), +1 of word i / 2
                    if (i & 1) {
                        pk_cur[i / 2] = pack2_f8<true>(p[0], p[1], pk_cur[i / 2]);
                    } else {
                        pk_cur[i / 2] = pack2_f8<false>(p[0], p[1], pk_cur[i / 2]);
                    }
                } else {
                    pk_cur[i] = pack2<Tag>(p[0], p[1]);
                }
            };
            // the pairs of one half (first = 0 or 4) that chunk c of a block takes care of
            auto silu_chunk = [&](int first, int c) {
#pragma unroll
                for (int i = c * 4 / NCH; i < (c + 1) * 4 / NCH; ++i) {
                    silu_pair(first + i);
                }
            };
            constexpr int LOOKAHEAD = NCH >= 4 ? 2 : 1;

            if constexpr (HAS_MASK && !F8) {
                if (do_silu) {
                    order_bias(mw_cur);
                }
            }
            if constexpr (K64) {
                // ---- both products on the 64-deep MFMA ----
                if (do_pv) {
                    const uint8_t* const v_lo = reinterpret_cast<const uint8_t*>(v_slot(std::integral_constant<int, LO>{}));
                    const uint8_t* const v_hi = reinterpret_cast<const uint8_t*>(v_slot(std::integral_constant<int, HI>{}));
                    const uint32_t(&p_lo)[8] = p_block(std::integral_constant<int, LO>{});
                    const uint32_t(&p_hi)[8] = p_block(std::integral_constant<int, HI>{});
                    constexpr int MT0 = PAR ? MTILES / 2 : 0;  // this step's half of the output tiles
                    // sub-tile t0 + 1 may lie past the end of the sweep: its P^T block is zero, and its slot then holds
                    // whatever an earlier sweep left there, so its half of the operand is zero as well
                    const bool hi_ok = INTERIOR || (t0 + 1 < x_end);
                    // V^T operand of output tile mt: keys of the two 16-key groups of either sub-tile, in P^T's order
                    auto read_v64 = [&](int mt, u32x4_t& lo, u32x4_t& hi) {
                        const u32x2_t a0 = lds_read_tr8_b64(v_lo + v_lane_off[mt]);
                        const u32x2_t a1 = lds_read_tr8_b64(v_lo + v_lane_off[mt] + 16 * D);
                        const u32x2_t b0 = lds_read_tr8_b64(v_hi + v_lane_off[mt]);
                        const u32x2_t b1 = lds_read_tr8_b64(v_hi + v_lane_off[mt] + 16 * D);
                        lo = u32x4_t{a0[0], a0[1], a1[0], a1[1]};
                        hi = u32x4_t{b0[0], b0[1], b1[0], b1[1]};
                    };
                    u32x4_t va_lo[NCH2], va_hi[NCH2];
                    read_v64(MT0, va_lo[0], va_hi[0]);
                    __builtin_amdgcn_sched_barrier(0);
                    const u32x4_t pb_lo = {p_lo[0], p_lo[1], p_lo[2], p_lo[3]};
                    const u32x4_t pb_hi = {p_hi[0], p_hi[1], p_hi[2], p_hi[3]};
#pragma unroll
                    for (int c = 0; c < NCH2; ++c) {
                        u32x4_t hi = va_hi[c];
                        if constexpr (!INTERIOR) {
                            if (!hi_ok) {
                                hi = u32x4_t{0u, 0u, 0u, 0u};
                            }
                        }
                        o_acc[MT0 + c] = mfma32x64_f8(va_lo[c], hi, pb_lo, pb_hi, o_acc[MT0 + c]);
                        if (c + 1 < NCH2) {
                            read_v64(MT0 + c + 1, va_lo[c + 1], va_hi[c + 1]);
                        }
#pragma unroll
                        for (int i = c * 4 / NCH2; i < (c + 1) * 4 / NCH2; ++i) {
                            silu_pair(i);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else if (do_silu) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        silu_pair(i);
                    }
                }
                if (do_qk) {
                    u32x4_t kop[KREADS];
                    kop[0] = read_k(0);
                    kop[1] = read_k(1);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int c = 0; c < NCH2; ++c) {
                        if (c == 0) {
                            f32x16_t zero;
#pragma unroll
                            for (int i = 0; i < 16; ++i) {
                                zero[i] = 0.f;
                            }
                            s_nxt = mfma32x64_f8(kop[0], kop[1], qf[0], qf[1], zero);
                        } else {
                            s_nxt = mfma32x64_f8(kop[2 * c], kop[2 * c + 1], qf[2 * c], qf[2 * c + 1], s_nxt);
                        }
                        if (c + 1 < NCH2) {
                            kop[2 * c + 2] = read_k(2 * c + 2);
                            kop[2 * c + 3] = read_k(2 * c + 3);
                        }
#pragma unroll
                        for (int i = c * 4 / NCH2; i < (c + 1) * 4 / NCH2; ++i) {
                            silu_pair(4 + i);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else if (do_silu) {
#pragma unroll
                    for (int i = 4; i < 8; ++i) {
                        silu_pair(i);
                    }
                }
            } else if (do_pv) {
                u32x4_t vop[NCH];
#pragma unroll
                for (int c = 0; c < LOOKAHEAD; ++c) {
                    vop[c] = read_v(c);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int c = 0; c < NCH; ++c) {
                    const int j2 = c % 2, mt = c / 2;
                    const u32x4_t pb = {pk_prev[4 * j2 + 0], pk_prev[4 * j2 + 1], pk_prev[4 * j2 + 2], pk_prev[4 * j2 + 3]};
                    o_acc[mt] = mfma32<Tag>(vop[c], pb, o_acc[mt]);
                    if (c + LOOKAHEAD < NCH) {
                        vop[c + LOOKAHEAD] = read_v(c + LOOKAHEAD);
                    }
                    silu_chunk(0, c);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else if (do_silu) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    silu_pair(i);
                }
            }
            if constexpr (HAS_RAB && !F8) {
                // the bias of sub-tile t + 2 (added to S^T(t + 2) at the end of the next step's QK block)
                __builtin_amdgcn_sched_barrier(0);
                if (INTERIOR || t + 2 < nx_w) {
                    load_rab(c0 + 64, rab_far);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (K64) {
                // (done above)
            } else if (do_qk) {
                u32x4_t kop[NCH];
#pragma unroll
                for (int c = 0; c < LOOKAHEAD; ++c) {
                    kop[c] = read_k(c);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int c = 0; c < NCH; ++c) {
                    if (c == 0) {
                        f32x16_t zero;
#pragma unroll
                        for (int i = 0; i < 16; ++i) {
                            zero[i] = 0.f;
                        }
                        s_nxt = mfma32<Tag>(kop[c], qf[c], zero);
                    } else {
                        s_nxt = mfma32<Tag>(kop[c], qf[c], s_nxt);
                    }
                    if (c + LOOKAHEAD < NCH) {
                        kop[c + LOOKAHEAD] = read_k(c + LOOKAHEAD);
                    }
                    silu_chunk(4, c);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if constexpr (HAS_RAB && !F8) {
                    // S^T(t+1) += rab^T, last so that the rab request has had the whole block to land
                    const u32x4_t r0 = {rab_nxt[0], rab_nxt[1], rab_nxt[2], rab_nxt[3]};
                    const u32x4_t r1 = {rab_nxt[4], rab_nxt[5], rab_nxt[6], rab_nxt[7]};
                    s_nxt = mfma32<Tag>(rab_route[0], r0, s_nxt);
                    s_nxt = mfma32<Tag>(rab_route[1], r1, s_nxt);
                }
            } else if (do_silu) {
#pragma unroll
                for (int i = 4; i < 8; ++i) {
                    silu_pair(i);
                }
            }
            // visibility: key c0 + 8*(e/4) + 4*lh + e%4 of element e is hidden at or past lim and inside the hole
            if (do_silu && !full && t >= static_cast<int>(rows_only & 0xffffu) && t < static_cast<int>(rows_only >> 16)) {
                // (a context row's limit lies at or past the end of the sub-tile, any other row's at or before its start)
                const uint32_t keep = lim_lane > c0 ? 0xffffffffu : 0u;
#pragma unroll
                for (int w = 0; w < (F8 ? 4 : 8); ++w) {
                    pk_cur[w] &= keep;
                }
            } else if (do_silu && !full) {
                constexpr int EPW = F8 ? 4 : 2;  // packed elements per word
#pragma unroll
                for (int w = 0; w < 16 / EPW; ++w) {
                    uint32_t keep = 0;
#pragma unroll
                    for (int e = 0; e < EPW; ++e) {
                        const int el = EPW * w + e;
                        const int kk = c0 + 8 * (el / 4) + (el % 4);  // + 4*lh is folded into the *_lane bounds
                        const bool vis = (kk < lim_lane) && !(kk >= hole_lo_lane && kk < hole_hi_lane);
                        const uint32_t bits = (F8 ? 0xffu : 0xffffu) << ((32 / EPW) * e);
                        keep |= vis ? bits : 0u;
                    }
                    pk_cur[w] &= keep;
                }
            }

            if constexpr (K64 && !INTERIOR) {
                // a step past the end of this wavefront's sweep: its P^T block may be the upper half of the last pair
                if (!do_silu) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        pk_cur[i] = 0u;
                    }
                }
            }

            if constexpr (kRequestsAtEnd) {
                __builtin_amdgcn_sched_barrier(0);
                tile_requests();
            }

            // (4) the requests made two time steps ago have landed (mine), then everybody's
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(K64 ? (PAR ? kWaitOdd64 : kWaitEven64) : kWaitTiles);
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
        };

        // ---- key sweep ----
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (x_end > x_begin) {
            // interior steps of this wavefront: [x_begin + 1, t_interior).  Sub-tile t + 1 (t + 2 with rab) must exist,
            // and sub-tile t must be fully visible: it ends at or before the smallest row limit and, when target
            // rows carve holes, before the first target key.  The wavefronts of a workgroup run different numbers
            // of interior steps; every step of either kind ends in the same one barrier, so the counts match.
            int t_interior = nx_w - (HAS_RAB ? 2 : 1);
            {
                int full_tiles = lim_min >> 5;
                if (any_hole) {
                    const int before_targets = hist_k > 0 ? hist_k >> 5 : 0;
                    full_tiles = full_tiles < before_targets ? full_tiles : before_targets;
                }
                t_interior = t_interior < full_tiles ? t_interior : full_tiles;
            }
            // (short sweeps stay on the general step: measured on MI355X, sweeps under about twenty steps gain nothing
            // from the second copy of the step and lose a little to fetching its instructions)
            if (x_end - x_begin < kInteriorMinSteps) {
                t_interior = -1;
            }
            typedef std::false_type general_t;
            typedef std::true_type interior_t;
            // (64-deep PV: the pair that holds the last sub-tile is consumed two and three steps after its first half)
            const int x_last = K64 ? x_end + 1 + (x_end & 1) : x_end;
            int t = x_begin - 1;
            while (true) {
                time_step(ic3_t{}, general_t{}, t);
                if (++t > x_last) {
                    break;
                }
                time_step(ic0_t{}, general_t{}, t);
                if (++t > x_last) {
                    break;
                }
                // (t mod 4 == 1 and t >= x_begin + 1 here; at head dim 256 a step is 32 MFMAs long and the general
                // step's overhead is small beside it, so that variant is not given the second copy)
                if constexpr (D <= 128) {
                    // (64-deep PV: the pair consumed in step t begins at t - 3, which must lie in this sweep)
                    while (t + 4 <= t_interior && (!K64 || t > x_begin + 1)) {
                        time_step(ic1_t{}, interior_t{}, t);
                        time_step(ic2_t{}, interior_t{}, t + 1);
                        time_step(ic3_t{}, interior_t{}, t + 2);
                        time_step(ic0_t{}, interior_t{}, t + 3);
                        t += 4;
                    }
                }
                time_step(ic1_t{}, general_t{}, t);
                if (++t > x_last) {
                    break;
                }
                time_step(ic2_t{}, general_t{}, t);
                if (++t > x_last) {
                    break;
                }
            }
        }

        // ---- split item: hand in this part; the part that completes the item adds all of them up ----
        bool store_rows = true;
        if constexpr (SPLIT) {
            if (n_parts > 1) {
                // The partial outputs travel between workgroups on different XCDs, whose L2 caches do not see each
                // other's lines: they are written and read with device-scope accesses (through to memory / from
                // memory), which costs nothing to anybody else, instead of writing back and invalidating whole caches
                // around the counter.  Order: stores complete (the wait the barrier brings) -> barrier -> count in.
                constexpr int kDeviceScope = 1 | 16;  // cache policy bits sc0 | sc1 of gfx94x / gfx950 buffer accesses
                constexpr int kQuads = MTILES * 4;                       // 16-byte pieces of a lane's accumulators
                constexpr uint32_t kPartBytes = kBlockM * D * 4u;        // one partial output
                const int ws_index = uniform(static_cast<int>(s_item[9]));
                const __amdgpu_buffer_rsrc_t ws_rsrc =
                    make_rsrc(reinterpret_cast<const uint8_t*>(a.ws) + static_cast<int64_t>(ws_index) * kPartBytes,
                              static_cast<uint32_t>(n_parts) * kPartBytes);
                // piece q of (wavefront, lane) sits at ((wave * kQuads + q) * 64 + lane) * 16 bytes: each store
                // instruction writes 1 KiB in a row
                const uint32_t lane_off = static_cast<uint32_t>(wave * kQuads * 64 + lane) * 16u;
                typedef __attribute__((ext_vector_type(4))) float f32x4_t;
#pragma unroll
                for (int q = 0; q < kQuads; ++q) {
                    // (the four floats are reinterpreted as one vector: element-wise reinterpretation into an integer
                    // vector is narrowed to the first element by the optimiser of this toolchain)
                    const f32x4_t v4 = {o_acc[q / 4][4 * (q % 4) + 0], o_acc[q / 4][4 * (q % 4) + 1],
                                        o_acc[q / 4][4 * (q % 4) + 2], o_acc[q / 4][4 * (q % 4) + 3]};
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, v4), ws_rsrc,
                                                           static_cast<int>(part * kPartBytes + lane_off + q * 1024u), 0,
                                                           kDeviceScope);
                }
                __builtin_amdgcn_s_waitcnt(0);
                __syncthreads();  // every wavefront's stores have completed
                unsigned int* const arrived = a.counters + kSplitCounterBase + s_item[8];
                if (tid == 0) {
                    s_item[10] = __hip_atomic_fetch_add(arrived, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                __syncthreads();
                store_rows = s_item[10] == static_cast<uint32_t>(n_parts - 1);
                if (store_rows) {
                    // the m partial outputs, added in part order whoever arrived last; the loads of one part
                    // are all in flight together
                    f32x4_t tot[kQuads];
#pragma unroll
                    for (int q = 0; q < kQuads; ++q) {
                        tot[q] = f32x4_t{0.f, 0.f, 0.f, 0.f};
                    }
                    for (int pp = 0; pp < n_parts; ++pp) {
                        u32x4_t got[kQuads];
#pragma unroll
                        for (int q = 0; q < kQuads; ++q) {
                            got[q] = __builtin_amdgcn_raw_buffer_load_b128(
                                ws_rsrc, static_cast<int>(pp * kPartBytes + lane_off + q * 1024u), 0, kDeviceScope);
                        }
#pragma unroll
                        for (int q = 0; q < kQuads; ++q) {
                            tot[q] += __builtin_bit_cast(f32x4_t, got[q]);
                        }
                    }
#pragma unroll
                    for (int q = 0; q < kQuads; ++q) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            o_acc[q / 4][4 * (q % 4) + e] = tot[q][e];
                        }
                    }
                }
                __syncthreads();  // s_item[10] has been read before the next fetch writes the item
            }
        }

        // ---- store O: lane holds query row (wr0 + ln), dims 32*mt + 8*g + 4*lh + 0..3 ----
        // Written as they lie in the registers, the rows would go out in 8-byte pieces, 16 store instructions
        // touching every 128-byte line of the tile; measured, these partial-line writes cost a 42 us launch 6 us.
        // So the wavefront passes its 32 rows through LDS (its own K slot of the ring, idle between two sweeps;
        // 16-byte chunks XOR-ed with the row so that neither side has bank conflicts to speak of) and writes them
        // 16 bytes per lane, whole lines per instruction.  (fp8 sub-tiles are half the size of the 16-bit output
        // rows: rows 0..15 go through the wavefront's K slot, rows 16..31 through its V slot.)
        const bool staged = a.out_vec_ok != 0;
        if (staged) {
            // every wavefront's tile requests have landed (the last ones, past the end, move nothing, but they
            // name the slots) before anybody writes a slot
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
        }
        if (store_rows && staged) {
            {
                uint16_t* const stage_lo = wave == 0 ? s_k0 : (wave == 1 ? s_k1 : (wave == 2 ? s_k2 : s_k3));
                uint16_t* const stage_hi = F8 ? (wave == 0 ? s_v0 : (wave == 1 ? s_v1 : (wave == 2 ? s_v2 : s_v3))) : stage_lo + 16 * D;
                constexpr int OCPR = D / 8;  // 16-byte chunks per staged row
                // the LDS offsets below depend on the lane only; opaque copies of the lane's coordinates keep the
                // compiler from working them out once, ahead of the item loop, and carrying two dozen registers
                // through the sweep, where there is none to spare
                int ln_e = ln, lh_e = lh, lane_e = lane;
                asm volatile("" : "+v"(ln_e), "+v"(lh_e), "+v"(lane_e));
#pragma unroll
                for (int mt = 0; mt < MTILES; ++mt) {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        u32x2_t w;
                        w[0] = pack2<OutTag>(o_acc[mt][4 * g + 0] * c_out, o_acc[mt][4 * g + 1] * c_out);
                        w[1] = pack2<OutTag>(o_acc[mt][4 * g + 2] * c_out, o_acc[mt][4 * g + 3] * c_out);
                        const int chunk = (4 * mt + g) ^ (ln_e & (OCPR - 1));
                        uint16_t* const row_at = (ln_e < 16 ? stage_lo : stage_hi) + (ln_e & 15) * D;
                        *reinterpret_cast<u32x2_t*>(row_at + chunk * 8 + 4 * lh_e) = w;
                    }
                }
                // (one wavefront: its LDS accesses execute in order; the fences keep the compiler from moving the reads up)
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                constexpr int RPI = 64 / OCPR;  // rows per store instruction
                constexpr int kNonTemporal = 2;  // cache policy bit nt: the rows are not read again by this kernel (measured: 1 - 4 % of a launch)
                const int rr = lane_e / OCPR;
                const int cc = lane_e % OCPR;
#pragma unroll
                for (int i = 0; i < 32 / RPI; ++i) {
                    const int r = i * RPI + rr;  // (the rows of one instruction lie in one half: RPI divides 16)
                    const uint16_t* const row_at = (i * RPI < 16 ? stage_lo : stage_hi) + (((i * RPI) & 15) + rr) * D;
                    const u32x4_t piece = *reinterpret_cast<const u32x4_t*>(row_at + (cc ^ (r & (OCPR - 1))) * 8);
                    const uint32_t off = (cc * 8 < a.d_v) ? static_cast<uint32_t>(wr0 + r) * o_stride + cc * 16u : kOutOfRange;
                    __builtin_amdgcn_raw_buffer_store_b128(piece, o_rsrc, static_cast<int>(off), 0, kNonTemporal);
                }
            }
        } else if (store_rows) {
            const uint32_t row_off = static_cast<uint32_t>(wr0 + ln) * o_stride;
#pragma unroll
            for (int mt = 0; mt < MTILES; ++mt) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int d0 = 32 * mt + 8 * g + 4 * lh;
                    const uint32_t off = (d0 < a.d_v) ? row_off + d0 * 2u : kOutOfRange;
                    u32x2_t w;
                    w[0] = pack2<OutTag>(o_acc[mt][4 * g + 0] * c_out, o_acc[mt][4 * g + 1] * c_out);
                    w[1] = pack2<OutTag>(o_acc[mt][4 * g + 2] * c_out, o_acc[mt][4 * g + 3] * c_out);
                    __builtin_amdgcn_raw_buffer_store_b64(w, o_rsrc, static_cast<int>(off), 0, 0);
                }
            }
        }

        // (the barriers of the sweep separate this item's reads of s_item from the next fetch)
        if constexpr (kStaticList) {
            ++round;
            __syncthreads();  // every wavefront has read its staged rows back before the next requests write the slots
        }
    }

    // ---- rows past the last offset: zero-fill ----
    {
        const int64_t first_tail = last_offset < 0 ? 0 : (last_offset < a.total_q ? last_offset : a.total_q);
        const int64_t row_elems = static_cast<int64_t>(n_heads) * a.d_v;
        const int64_t n_tail = (a.total_q - first_tail) * row_elems;
        uint16_t* tail = out16 + first_tail * row_elems;
        for (int64_t e = static_cast<int64_t>(blockIdx.x) * kThreads + tid; e < n_tail;
             e += static_cast<int64_t>(gridDim.x) * kThreads) {
            tail[e] = 0;
        }
    }

}

}  // namespace hstu
