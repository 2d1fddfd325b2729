// in_linear_silu forward for gfx950: mixed = x @ weight^T + bias; linear_output = mixed (rounded to the input type);
// (user, value, query, key) = split(silu(linear_output), split sizes, last dim).
//
// Follows the reference's kernel in what is rounded where: the product is accumulated in fp32 with the fp32 bias, the
// sum is rounded once to the 16-bit type (that is linear_output), and SiLU is taken in fp32 of that rounded value and
// rounded to nearest even (ascendc/activation/in_linear_silu/in_linear_silu_forward/op_kernel/in_linear_silu_kernel.h:80-109,
// block_epilogue_elemwise_split.h:160-183, tile_elemwise_silu.h:36-47: x / (1 + exp(-x))).
//
// What bounds it: every output element is written twice (linear_output and its split) = 4 bytes of HBM writes against
// 2k flops, and the reference's shapes have k = 16..256 against n = 1024..16384: HBM-write-bound up to k of a few
// hundred.  So the kernel is laid out around its stores: the weight rows are the A operand of the 32x32x16 MFMA and
// the x rows the B operand, which leaves a lane with the outputs of ONE x row, and the weight rows of a 32-row block
// are placed in LDS in a permuted order so that those outputs are 2 x 8 CONSECUTIVE columns: 16-byte pieces, which
// the epilogue passes through LDS so that every store instruction writes whole 128-byte lines of an output row.
//
// Tile: 128 x rows by 128 weight rows per workgroup (4 wavefronts, 64 x 64 each = 4 accumulator blocks), k in steps
// of 32 through a ring of STAGES tiles in LDS filled by direct-to-LDS loads (16 KB per stage: 256 rows of 64 bytes,
// chunk index XOR-ed with (row / 4) % 4 so that the 16-byte operand reads of 16 consecutive rows fall into 16
// different bank groups).  STAGES = 2 (36 KB with the epilogue's staging: four workgroups per CU overlap their load /
// product / store phases) 3 (48 KB, three workgroups per CU, prefetch distance 2) or 4 (64 KB, two); the host picks by k.
#pragma once
#include "hstu_fwd_kernel.hip.h"

namespace hstu {

constexpr int kIlsThreads = 256;
constexpr int kIlsTileM = 128;  // x rows per workgroup
constexpr int kIlsStepK = 32;
constexpr int kIlsXcds = 8;  // MI355X: 8 XCDs, workgroups dealt round-robin

// MFMA row r of a 32-row block of weight rows -> column offset within the block, chosen so that the 16 accumulator
// values of a lane (rows 8g + 4h + j, g = 0..3, j = 0..3, h = lane / 32) are columns 16(g/2) + 8h + 4(g%2) + j:
// two runs of 8 consecutive columns (16 bytes each on the way to the staging rows of the epilogue)
__device__ __forceinline__ int ils_column_of_mfma_row(int r)
{
    const int g = r >> 3, h = (r >> 2) & 1, j = r & 3;
    return 16 * (g >> 1) + 8 * h + 4 * (g & 1) + j;
}

// the two values of a packed pair of the 16-bit type, as floats
template <typename Tag>
__device__ __forceinline__ void ils_unpack2(uint32_t w, float& lo, float& hi);
template <>
__device__ __forceinline__ void ils_unpack2<bf16_tag>(uint32_t w, float& lo, float& hi)
{
    lo = __builtin_bit_cast(float, w << 16);
    hi = __builtin_bit_cast(float, w & 0xffff0000u);
}
template <>
__device__ __forceinline__ void ils_unpack2<f16_tag>(uint32_t w, float& lo, float& hi)
{
    typedef __attribute__((ext_vector_type(2))) _Float16 pair_t;
    const pair_t r = __builtin_bit_cast(pair_t, w);
    lo = static_cast<float>(r[0]);
    hi = static_cast<float>(r[1]);
}

// x / (1 + exp(-x)) with the hardware's exp2 and reciprocal (1 ulp each; the result is rounded to 8 or 11 bits).
// The epilogue is what the vector unit spends its time on -- 4 bytes of output per element leave room for about 25
// vector instruction slots per element before the kernel stops being bound by its stores, and an IEEE division alone
// costs 10 -- so it is kept to an add, a conversion, two multiplies, an add and the two transcendental instructions.
__device__ __forceinline__ float ils_silu(float v)
{
    const float t = __builtin_amdgcn_exp2f(v * -1.4426950408889634f);
    return v * __builtin_amdgcn_rcpf(1.0f + t);
}

// workgroups per CU a variant is compiled for (registers and LDS)
constexpr int ils_workgroups_per_cu(int stages, int wnb) { return wnb == 4 ? 2 : (stages == 2 ? 4 : (stages == 3 ? 3 : 2)); }

// WNB = 32-row weight blocks per wavefront: 2 (tile 128 x 128, 64 accumulator registers) or 4 (tile 128 x 256,
// 128 accumulator registers: twice the MFMAs per k step and per byte staged, for the shapes bound by the products)
template <typename Tag, int STAGES, int WNB = 2>
__global__ __launch_bounds__(kIlsThreads, ils_workgroups_per_cu(STAGES, WNB)) void in_linear_silu_kernel(const InLinearSiluArgs a)
{
    constexpr int kIlsTileN = 64 * WNB;  // weight rows (output columns) per workgroup: 2 wavefronts x WNB blocks of 32
    constexpr int kReqs = (kIlsTileM + kIlsTileN) / 16 / 4;  // direct-to-LDS instructions per wavefront and stage
    constexpr int kReqsW = kIlsTileN / 16 / 4;               // of which for weight rows (the first ones)
    constexpr int kStageElems = (kIlsTileM + kIlsTileN) * kIlsStepK;  // 16-bit elements per stage
    // the epilogue stages both results of 32 x rows by 64 columns per wavefront in the same memory
    constexpr int kEpiRowElems = 64 + 8;
    constexpr int kEpiWaveElems = 2 * 32 * kEpiRowElems;
    constexpr int kLdsElems = STAGES * kStageElems > 4 * kEpiWaveElems ? STAGES * kStageElems : 4 * kEpiWaveElems;
    __shared__ __attribute__((aligned(1024))) uint16_t s_tiles[kLdsElems];

    const int lane = threadIdx.x & 63;
    const int wave = uniform(threadIdx.x >> 6);
    const int n_tiles_n = (a.n + kIlsTileN - 1) / kIlsTileN;
    // Tile order.  Plain: n tiles fastest, so the workgroups in flight write whole output rows between them.  Grouped
    // (a.xcd_groups, chosen by the host for a weight matrix that every L2 can hold beside its streams): workgroup b runs
    // on XCD b % 8, each with an L2 of its own; blocks are dealt in groups of 8 m tiles, XCD j taking all n tiles of the
    // j-th m tile of the group, so that an x tile is fetched by one XCD only.  Measured at m = 20292 (plain -> grouped):
    // n 2048, k 512: fetched bytes 169 -> 38 MB at the same 71 us; n 1024, k 256: 27.7 -> 24.2 us; n 2048, k 128: 41 -> 38 us;
    // larger weights lose (n 8192, k 2048: 568 -> 661 us; n 32768, k 8192: 4.8 -> 6.1 ms), and so does k = 64 (110 -> 116 us).
    // The grid is padded to whole groups; workgroups past the end leave at once.
    int tile_m, tile_n;
    if (a.xcd_groups) {
        const int group = blockIdx.x / (kIlsXcds * n_tiles_n);
        const int in_group = blockIdx.x - group * (kIlsXcds * n_tiles_n);
        tile_m = group * kIlsXcds + (in_group % kIlsXcds);
        tile_n = in_group / kIlsXcds;
    } else {
        tile_m = blockIdx.x / n_tiles_n;
        tile_n = blockIdx.x - tile_m * n_tiles_n;
    }
    if (static_cast<int64_t>(tile_m) * kIlsTileM >= a.m) {
        return;
    }
    const int64_t m0 = static_cast<int64_t>(tile_m) * kIlsTileM;
    const int n0 = tile_n * kIlsTileN;
    const int rows_w = min(kIlsTileN, a.n - n0);
    const int rows_x = a.m - m0 < kIlsTileM ? static_cast<int>(a.m - m0) : kIlsTileM;
    const uint32_t row_bytes = static_cast<uint32_t>(a.k) * 2u;
    // rows past the end of the matrices read as zeros (out-of-range bytes of a buffer descriptor)
    const __amdgpu_buffer_rsrc_t w_rsrc =
        make_rsrc(static_cast<const uint8_t*>(a.weight) + static_cast<int64_t>(n0) * row_bytes, rows_w * row_bytes);
    const __amdgpu_buffer_rsrc_t x_rsrc =
        make_rsrc(static_cast<const uint8_t*>(a.x) + m0 * row_bytes, rows_x * row_bytes);

    // ---- requests: a stage is LDS rows of 64 bytes (the tile's weight rows, then its 128 x rows); one direct-to-LDS
    // instruction of a wavefront fills 16 rows (lane -> row lane / 4, physical chunk lane % 4); the instructions of
    // a stage are dealt round-robin to the 4 wavefronts
    uint32_t req_off[kReqs];   // byte offset of the lane's source row (+ logical chunk) for k = 0
    int req_chunk[kReqs];      // logical 16-byte chunk (0..3) the lane fetches
#pragma unroll
    for (int i = 0; i < kReqs; ++i) {
        const int q = wave + 4 * i;               // instruction of the stage
        const int lds_row = 16 * q + (lane >> 2);
        const int chunk = (lane & 3) ^ ((lds_row >> 2) & 3);
        // the first kReqsW instructions of a wavefront fill weight rows, the others x rows
        const int src_row = i < kReqsW ? (lds_row & ~31) + ils_column_of_mfma_row(lds_row & 31) : lds_row - kIlsTileN;
        req_chunk[i] = chunk;
        req_off[i] = static_cast<uint32_t>(src_row) * row_bytes + chunk * 16u;
    }
    auto request = [&](int stage, int step) {
        const int k0 = step * kIlsStepK;
        uint16_t* base = s_tiles + stage * kStageElems;
#pragma unroll
        for (int i = 0; i < kReqs; ++i) {
            const int q = wave + 4 * i;
            // chunks past the end of a row must read as zeros: they would otherwise be the next row's first values
            const bool in_row = k0 + 8 * req_chunk[i] < a.k;
            const uint32_t off = in_row ? req_off[i] + static_cast<uint32_t>(k0) * 2u : kOutOfRange;
            load_to_lds_b128(i < kReqsW ? w_rsrc : x_rsrc, base + q * 16 * kIlsStepK, off);
        }
    };

    // ---- operand reads: wavefront (wm, wn) owns x rows 64 wm .. +64 and weight rows 32 WNB wn .. +32 WNB of the tile
    const int wm = wave >> 1, wn = wave & 1;
    int a_off[WNB], b_off[2];  // element offsets within a stage of the lane's row of each 32-row block, k chunk 0
    const int r = lane & 31, half = lane >> 5;
#pragma unroll
    for (int blk = 0; blk < WNB; ++blk) {
        a_off[blk] = (32 * WNB * wn + 32 * blk + r) * kIlsStepK;
    }
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
        b_off[blk] = (kIlsTileN + 64 * wm + 32 * blk + r) * kIlsStepK;
    }
    const int swz = (r >> 2) & 3;  // the same for all the rows above: they differ by multiples of 32

    f32x16_t acc[WNB][2];  // [weight block][x block]
#pragma unroll
    for (int i = 0; i < WNB; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                acc[i][j][e] = 0.0f;
            }
        }
    }

    const int n_steps = (a.k + kIlsStepK - 1) / kIlsStepK;
    constexpr int kAhead = STAGES - 1;
    for (int s = 0; s < kAhead && s < n_steps; ++s) {
        request(s, s);
    }
    constexpr int kWait0 = 0 | (7 << 4) | (15 << 8);
    constexpr int kWait4 = kReqs | (7 << 4) | (15 << 8);
    constexpr int kWait8 = 2 * kReqs | (7 << 4) | (15 << 8);
    static_assert(2 * kReqs <= 15, "the count must fit the low bits of the wait instruction");
    for (int t = 0; t < n_steps; ++t) {
        // requests issued after step t's own: steps t+1 .. t+STAGES-2 (kReqs instructions each)
        const int later = min(STAGES - 2, n_steps - 1 - t);
        __builtin_amdgcn_sched_barrier(0);
        if (later >= 2) {
            __builtin_amdgcn_s_waitcnt(kWait8);
        } else if (later == 1) {
            __builtin_amdgcn_s_waitcnt(kWait4);
        } else {
            __builtin_amdgcn_s_waitcnt(kWait0);
        }
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        // every wavefront is past step t-1: its stage may be overwritten
        if (t + kAhead < n_steps) {
            request((t + kAhead) % STAGES, t + kAhead);
        }
        const uint16_t* st = s_tiles + (t % STAGES) * kStageElems;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            const int chunk = ((2 * kk + half) ^ swz) * 8;
            u32x4_t wa[WNB], xb[2];
#pragma unroll
            for (int blk = 0; blk < WNB; ++blk) {
                wa[blk] = *reinterpret_cast<const u32x4_t*>(st + a_off[blk] + chunk);
            }
#pragma unroll
            for (int blk = 0; blk < 2; ++blk) {
                xb[blk] = *reinterpret_cast<const u32x4_t*>(st + b_off[blk] + chunk);
            }
#pragma unroll
            for (int i = 0; i < WNB; ++i) {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    acc[i][j] = mfma32<Tag>(wa[i], xb[j], acc[i][j]);
                }
            }
        }
    }

    // ---- epilogue.  A lane holds, for its x row (lane % 32) of each x block, 2 runs of 8 consecutive columns per
    // weight block.  Stored from there, a 128-byte line of an output row would be written in four pieces by four
    // instructions; with both outputs in flight the partly written lines overflow the L2 and go to memory piecewise
    // (measured: both outputs together took 4x the sum of each alone).  So the two 16-bit results of 32 x rows are
    // staged through LDS (rows padded to 144 bytes: 16-byte writes of consecutive rows and the 128-byte row reads
    // both spread over the banks) and written back with 8 lanes per row: every store instruction writes 8 whole lines.
    const int split1 = a.split_end[0], split2 = a.split_end[1], split3 = a.split_end[2];
    __builtin_amdgcn_s_barrier();  // every wavefront is done reading the last stage
    uint16_t* staged = s_tiles + wave * kEpiWaveElems;
    const int out_row = lane >> 3, out_chunk = lane & 7;
    // the wavefront's columns go out 64 at a time (two weight blocks): WNB / 2 rounds
#pragma unroll
    for (int ch = 0; ch < WNB / 2; ++ch) {
        const int col0 = n0 + 32 * WNB * wn + 64 * ch;  // first column of this round
        const int out_col = col0 + 8 * out_chunk;      // first of the lane's 8 columns when it writes back
        // the split these 8 columns belong to (split sizes are multiples of 16, the 8 columns are aligned to 8)
        uint16_t* split_base;
        int split_cols, split_col;
        if (out_col < split1) {
            split_base = static_cast<uint16_t*>(a.user), split_cols = split1, split_col = out_col;
        } else if (out_col < split2) {
            split_base = static_cast<uint16_t*>(a.value), split_cols = split2 - split1, split_col = out_col - split1;
        } else if (out_col < split3) {
            split_base = static_cast<uint16_t*>(a.query), split_cols = split3 - split2, split_col = out_col - split2;
        } else {
            split_base = static_cast<uint16_t*>(a.key), split_cols = a.n - split3, split_col = out_col - split3;
        }
        float bias[2][2][8];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int run = 0; run < 2; ++run) {
                const int col = col0 + 32 * i + 16 * run + 8 * half;
                const bool have = a.bias != nullptr && col < a.n;
                const float4 b0 = have ? *reinterpret_cast<const float4*>(a.bias + col) : make_float4(0.f, 0.f, 0.f, 0.f);
                const float4 b1 = have ? *reinterpret_cast<const float4*>(a.bias + col + 4) : make_float4(0.f, 0.f, 0.f, 0.f);
                bias[i][run][0] = b0.x, bias[i][run][1] = b0.y, bias[i][run][2] = b0.z, bias[i][run][3] = b0.w;
                bias[i][run][4] = b1.x, bias[i][run][5] = b1.y, bias[i][run][6] = b1.z, bias[i][run][7] = b1.w;
            }
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
#pragma unroll
                for (int run = 0; run < 2; ++run) {
                    // accumulator element 8 * run + e is MFMA row 8g + 4h + (e % 4) with g = 2 * run + e / 4: column
                    // 32 i + 16 run + 8 h + e of the round's 64.  linear_output = the sum rounded once; SiLU is taken
                    // of the rounded value, as in the reference.
                    u32x4_t lin, out;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        lin[e] = pack2<Tag>(acc[2 * ch + i][j][8 * run + 2 * e] + bias[i][run][2 * e],
                                            acc[2 * ch + i][j][8 * run + 2 * e + 1] + bias[i][run][2 * e + 1]);
                        float lo, hi;
                        ils_unpack2<Tag>(lin[e], lo, hi);
                        out[e] = pack2<Tag>(ils_silu(lo), ils_silu(hi));
                    }
                    uint16_t* at = staged + r * kEpiRowElems + 32 * i + 16 * run + 8 * half;
                    *reinterpret_cast<u32x4_t*>(at) = lin;
                    *reinterpret_cast<u32x4_t*>(at + 32 * kEpiRowElems) = out;
                }
            }
            // the wavefront's own lanes wrote what its lanes now read: LDS keeps a wavefront's accesses in order; the
            // fence keeps the compiler from moving the reads up
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int row_in_block = 8 * q + out_row;
                const int64_t row = m0 + 64 * wm + 32 * j + row_in_block;
                const uint16_t* from = staged + row_in_block * kEpiRowElems + 8 * out_chunk;
                const u32x4_t lin = *reinterpret_cast<const u32x4_t*>(from);
                const u32x4_t out = *reinterpret_cast<const u32x4_t*>(from + 32 * kEpiRowElems);
                if (row < a.m && out_col < a.n) {
                    // (streaming stores: the outputs are not read again by this kernel, and kept out of the L2's way
                    // they leave the weights and the x tiles there -- 3 to 15 % faster over k = 64 .. 1024)
                    __builtin_nontemporal_store(lin, reinterpret_cast<u32x4_t*>(static_cast<uint16_t*>(a.linear_output) + row * a.n + out_col));
                    __builtin_nontemporal_store(out, reinterpret_cast<u32x4_t*>(split_base + row * split_cols + split_col));
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    }
}

}  // namespace hstu
