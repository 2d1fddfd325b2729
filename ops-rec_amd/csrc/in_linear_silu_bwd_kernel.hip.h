// The element-wise stage of in_linear_silu's backward for gfx950:
//
//   d_mixed = cat(user_grad, value_grad, query_grad, key_grad) * silu'(linear_output),
//   silu'(z) = s (1 + z (1 - s)),  s = sigmoid(z);        bias_grad = column sums of d_mixed
//
// (formula of the reference's backward golden,
//  ascendc/activation/in_linear_silu/in_linear_silu_backward/test/pytest/test_in_linear_silu_backward.py:120-135).
// d_mixed is what the two products of the linear layer's backward take (d x = d_mixed @ weight, d weight = d_mixed^T @ x):
// those are plain matrix products and stay with the caller's BLAS.
//
// Bound: HBM.  Per element 2 bytes of linear_output and 2 of a gradient are read and 2 of d_mixed written.  A lane owns
// 8 consecutive columns (16 bytes: split sizes are multiples of 16, so a lane's columns lie in one gradient tensor); a
// wavefront covers 1 KB of a row; a workgroup of 64 column lanes x 4 row lanes walks 64 rows of 512 columns, its
// column sums in registers.  The sums of the 4 row lanes are added through LDS and written as one partial row per
// workgroup; a second small kernel adds the partial rows in a fixed order (no atomics: the same bits every launch).
#pragma once
#include "in_linear_silu_kernel.hip.h"

namespace hstu {

constexpr int kIlsBwdThreads = 256;
constexpr int kIlsBwdRows = 64;    // rows per workgroup
constexpr int kIlsBwdCols = 512;   // columns per workgroup (64 lanes x 8)

template <typename Tag>
__global__ __launch_bounds__(kIlsBwdThreads) void in_linear_silu_dmixed_kernel(const InLinearSiluBwdArgs a)
{
    __shared__ float s_sums[4][kIlsBwdCols];
    const int col_lane = threadIdx.x & 63, row_lane = threadIdx.x >> 6;
    // one grid dimension, column blocks fastest: the workgroups in flight write whole rows between them
    const int col_blocks = (a.n + kIlsBwdCols - 1) / kIlsBwdCols;
    const int row_block = blockIdx.x / col_blocks;
    const int col_block = blockIdx.x - row_block * col_blocks;
    const int col = col_block * kIlsBwdCols + col_lane * 8;
    const int64_t row0 = static_cast<int64_t>(row_block) * kIlsBwdRows;
    const bool in_cols = col < a.n;
    const uint16_t* grad = nullptr;
    int grad_cols = 0, grad_col = 0;
    if (in_cols) {
        if (col < a.split_end[0]) {
            grad = static_cast<const uint16_t*>(a.user_grad), grad_cols = a.split_end[0], grad_col = col;
        } else if (col < a.split_end[1]) {
            grad = static_cast<const uint16_t*>(a.value_grad), grad_cols = a.split_end[1] - a.split_end[0],
            grad_col = col - a.split_end[0];
        } else if (col < a.split_end[2]) {
            grad = static_cast<const uint16_t*>(a.query_grad), grad_cols = a.split_end[2] - a.split_end[1],
            grad_col = col - a.split_end[1];
        } else {
            grad = static_cast<const uint16_t*>(a.key_grad), grad_cols = a.n - a.split_end[2], grad_col = col - a.split_end[2];
        }
    }
    float sums[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        sums[e] = 0.0f;
    }
    if (in_cols) {
        const uint16_t* lin = static_cast<const uint16_t*>(a.linear_output);
        uint16_t* out = static_cast<uint16_t*>(a.d_mixed);
#pragma unroll 4
        for (int i = 0; i < kIlsBwdRows / 4; ++i) {
            const int64_t row = row0 + 4 * i + row_lane;
            if (row < a.m) {
                const u32x4_t z4 = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(lin + row * a.n + col));
                const u32x4_t g4 =
                    __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(grad + row * grad_cols + grad_col));
                u32x4_t d4;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float z[2], g[2], d[2];
                    ils_unpack2<Tag>(z4[e], z[0], z[1]);
                    ils_unpack2<Tag>(g4[e], g[0], g[1]);
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const float s = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(z[h] * -1.4426950408889634f));
                        d[h] = g[h] * (s * (1.0f + z[h] * (1.0f - s)));
                        sums[2 * e + h] += d[h];
                    }
                    d4[e] = pack2<Tag>(d[0], d[1]);
                }
                __builtin_nontemporal_store(d4, reinterpret_cast<u32x4_t*>(out + row * a.n + col));
            }
        }
    }
    if (a.partial_sums == nullptr) {
        return;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        s_sums[row_lane][col_lane * 8 + e] = sums[e];
    }
    __syncthreads();
    // 256 threads, 512 columns: two columns each, the four row lanes added in a fixed order
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int c = threadIdx.x + j * kIlsBwdThreads;
        const int gc = col_block * kIlsBwdCols + c;
        if (gc < a.n) {
            a.partial_sums[static_cast<int64_t>(row_block) * a.n + gc] =
                (s_sums[0][c] + s_sums[1][c]) + (s_sums[2][c] + s_sums[3][c]);
        }
    }
}

// bias_grad[c] = sum over the partial rows.  A workgroup owns 32 columns; its 8 row lanes each add every 8th partial
// row (8 independent loads in flight per lane), and the 8 lane sums are added in lane order: a fixed order, whatever
// the timing.
constexpr int kIlsBiasCols = 32;
constexpr int kIlsBiasLanes = 8;

__global__ __launch_bounds__(kIlsBiasCols* kIlsBiasLanes) void in_linear_silu_bias_grad_kernel(
    const float* partial_sums, float* bias_grad, int n_partials, int n)
{
    __shared__ float s_lane[kIlsBiasLanes][kIlsBiasCols];
    const int col_lane = threadIdx.x % kIlsBiasCols, row_lane = threadIdx.x / kIlsBiasCols;
    const int c = blockIdx.x * kIlsBiasCols + col_lane;
    float total = 0.0f;
    if (c < n) {
        int p = row_lane;
        for (; p + 7 * kIlsBiasLanes < n_partials; p += 8 * kIlsBiasLanes) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                v[u] = partial_sums[static_cast<int64_t>(p + u * kIlsBiasLanes) * n + c];
            }
            total += ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
        }
        for (; p < n_partials; p += kIlsBiasLanes) {
            total += partial_sums[static_cast<int64_t>(p) * n + c];
        }
    }
    s_lane[row_lane][col_lane] = total;
    __syncthreads();
    if (row_lane == 0 && c < n) {
        float sum = s_lane[0][col_lane];
#pragma unroll
        for (int l = 1; l < kIlsBiasLanes; ++l) {
            sum += s_lane[l][col_lane];
        }
        bias_grad[c] = sum;
    }
}

}  // namespace hstu
