// HSTU jagged attention backward for gfx950: the inputs the tuned backward kernels do not take.
//
// The reference's backward accepts what its forward accepts: bf16 / fp16 / fp32, any q/k head dim in [1, 512], any
// v head dim in [16, 512] in steps of 16 (ascendc/attention/hstu_v1/hstu_backward_v1/op_host, same tiling limits as
// hstu_forward_v1/op_host/tiling_policy.cpp:68-93).  The MFMA kernels of hstu_bwd_kernel.hip.h are built for bf16 /
// fp16 with head dims up to 256 and a q/k head dim that is a multiple of 8.  These two kernels cover the rest, the
// way hstu_fwd_generic_kernel covers it for the forward: plain fp32 arithmetic on the vector unit, written for
// coverage, not for speed, with the same formulas
//   X = alpha (Q K^T + rab),  sig = sigmoid(X),  P = X sig scale M,
//   dV = P^T dO,  dP = dO V^T,  dS = alpha scale M dP sig (1 + X (1 - sig)),  d rab = dS,  dQ = dS K,  dK = dS^T Q
// (hstu_backward_v1/op_kernel/vector_score.h:159-205) and the same split into two kernels without atomics: every
// output row is written by exactly one thread group, so the results are bit-reproducible.  P and dS are not rounded
// to the input type before the products that consume them.
//
//   hstu_bwd_generic_dq_kernel   one workgroup per 128-row query tile of one (sequence, head), 16 rows at a time:
//                                thread (r, c) computes dS of row r and key c of a 16-key tile from fp32 copies of
//                                the Q, dO, K and V rows in LDS, stores it as d rab when that is asked for, and
//                                then owns the columns c, c + 16, ... of dQ[r].
//   hstu_bwd_generic_dkv_kernel  one workgroup per 128-key tile of one (sequence, K/V head), 16 keys at a time:
//                                thread (kr, c) computes P and dS of key kr and query row c of a 16-row tile, for
//                                every query head of the group in turn, and owns the columns c, c + 16, ... of
//                                dK[kr] and dV[kr].
// The host clears dq, dk, dv and d rab ahead of the two launches: what no thread writes (rows of no sequence, rows
// past max_seq_len, bias elements outside the sequences or hidden by the mask) is zero.
#pragma once
#include "hstu_bwd_kernel.hip.h"
#include "hstu_fwd_generic_kernel.hip.h"

namespace hstu {

constexpr int kGenericBwdRows = 16;  // rows (query rows or keys) of a pass, and of a tile

// The kernels are instantiated for head dims up to MAXD = 128, 256 and 512: the four staged blocks take
// 4 x 16 x (MAXD + 4) floats of LDS (34 / 67 / 132 KB), so the smaller the bound the more workgroups share a CU and
// hide each other's load latency (a workgroup waits for its loads at every block: nothing is double-buffered here).

// 16 rows of `dim` elements, starting at row `row0` of a [*, row_elems] matrix at column `col0`, as floats into `dst`
// (row stride `stride`), zero beyond `n_rows` and up to `dim_padded`; thread t takes row t / 16, columns t % 16 + 16 i
template <typename T>
__device__ __forceinline__ void generic_stage_rows(float* dst, int stride, const void* src, int64_t first_row,
                                                   int64_t row_elems, int64_t col0, int row0, int n_rows, int dim,
                                                   int dim_padded, int tid)
{
    const int rr = tid >> 4;
    const int row = row0 + rr;
    const bool in = row < n_rows;
    const int64_t at = (first_row + row) * row_elems + col0;
    for (int dd = tid & 15; dd < dim_padded; dd += 16) {
        dst[rr * stride + dd] = (in && dd < dim) ? generic_load<T>(src, at + dd) : 0.0f;
    }
}

__device__ __forceinline__ float generic_dot(const float* x, const float* y, int n4)
{
    typedef __attribute__((ext_vector_type(4))) float f32x4_t;
    const f32x4_t* x4 = reinterpret_cast<const f32x4_t*>(x);
    const f32x4_t* y4 = reinterpret_cast<const f32x4_t*>(y);
    f32x4_t s4 = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int i = 0; i < n4; ++i) {
        s4 += x4[i] * y4[i];
    }
    return (s4[0] + s4[1]) + (s4[2] + s4[3]);
}

template <typename T, int MAXD>
__global__ __launch_bounds__(256) void hstu_bwd_generic_dq_kernel(const BwdArgs a)
{
    constexpr int RB = kGenericBwdRows, KB = kGenericBwdRows, kStride = MAXD + 4, kCols = MAXD / 16;
    __shared__ __attribute__((aligned(16))) float s_q[RB * kStride];
    __shared__ __attribute__((aligned(16))) float s_g[RB * kStride];
    __shared__ __attribute__((aligned(16))) float s_k[KB * kStride];
    __shared__ __attribute__((aligned(16))) float s_v[KB * kStride];
    __shared__ float s_ds[RB][KB + 1];

    const int tid = threadIdx.x;
    const int per_level = a.n_batch * a.n_heads_q;
    const int lvl = blockIdx.x / per_level;
    const int rem = blockIdx.x - lvl * per_level;
    const int qt = a.n_qtiles - 1 - lvl;
    const int b = rem / a.n_heads_q;
    const int h = rem - b * a.n_heads_q;
    const int hk = h / a.head_ratio;
    const SeqInfo si = load_seq(a, b);
    const int sq = si.sq, sk = si.sk;
    const int r0 = qt * kBlockM;
    if (r0 >= sq) {
        return;
    }
    const int64_t q_row_elems = static_cast<int64_t>(a.n_heads_q) * a.d_qk;
    const int64_t g_row_elems = static_cast<int64_t>(a.n_heads_q) * a.d_v;
    const int64_t k_row_elems = static_cast<int64_t>(a.n_heads_k) * a.d_qk;
    const int64_t v_row_elems = static_cast<int64_t>(a.n_heads_k) * a.d_v;
    const int64_t bias_plane = (static_cast<int64_t>(b) * a.n_heads_q + h) * a.max_q * static_cast<int64_t>(a.max_k);
    const int r = tid >> 4, c = tid & 15;
    const int d_qk4 = (a.d_qk + 3) & ~3;
    T* const dq_out = static_cast<T*>(a.dq);
    T* const drab_out = static_cast<T*>(a.drab);

    for (int pass = 0; pass < kBlockM / RB; ++pass) {
        const int rb = r0 + pass * RB;
        if (rb >= sq) {
            break;  // (the same for every thread)
        }
        const int row = rb + r;
        const bool row_in = row < sq;
        int lim, hole_lo, hole_hi;
        row_bounds(si, a.mask_type, a.target_group, row_in ? row : sq - 1, lim, hole_lo, hole_hi);
        // keys any of the 16 rows can see
        int kmax = sk;
        if (a.mask_type == 0) {
            const int last_row = (rb + RB < sq ? rb + RB : sq) - 1;
            kmax = last_row + si.delta + 1;
            if (rb < si.n_ctx) {
                kmax = kmax > si.hist_k ? kmax : si.hist_k;
            }
            kmax = kmax < 0 ? 0 : (kmax > sk ? sk : kmax);
        }
        __syncthreads();  // the previous pass is done with s_q / s_g
        generic_stage_rows<T>(s_q, kStride, a.q, si.q0, q_row_elems, static_cast<int64_t>(h) * a.d_qk, rb, sq, a.d_qk, d_qk4, tid);
        generic_stage_rows<T>(s_g, kStride, a.grad, si.q0, g_row_elems, static_cast<int64_t>(h) * a.d_v, rb, sq, a.d_v, a.d_v, tid);
        float dq[kCols];
#pragma unroll
        for (int j = 0; j < kCols; ++j) {
            dq[j] = 0.0f;
        }
        for (int kt = 0; kt * KB < kmax; ++kt) {
            const int key0 = kt * KB;
            __syncthreads();  // the previous tile's products are done (and s_q / s_g are written)
            generic_stage_rows<T>(s_k, kStride, a.k, si.k0, k_row_elems, static_cast<int64_t>(hk) * a.d_qk, key0, sk, a.d_qk, d_qk4, tid);
            generic_stage_rows<T>(s_v, kStride, a.v, si.k0, v_row_elems, static_cast<int64_t>(hk) * a.d_v, key0, sk, a.d_v, a.d_v, tid);
            __syncthreads();
            const int key = key0 + c;
            float ds = 0.0f;
            if (row_in && key < lim && !(key >= hole_lo && key < hole_hi)) {
                float s = generic_dot(s_q + r * kStride, s_k + c * kStride, d_qk4 / 4);
                const float dp = generic_dot(s_g + r * kStride, s_v + c * kStride, a.d_v / 4);
                const int64_t at = bias_plane + static_cast<int64_t>(row) * a.max_k + key;
                if (a.rab != nullptr) {
                    s += generic_load<T>(a.rab, at);
                }
                const float x = s * a.alpha;
                const float sig = 1.0f / (1.0f + __expf(-x));
                ds = a.alpha * a.scale * dp * sig * (1.0f + x * (1.0f - sig));
                if (a.mask_type == 3) {
                    ds *= generic_load<T>(a.mask, at);
                }
                if (drab_out != nullptr) {
                    drab_out[at] = static_cast<T>(ds);
                }
            }
            s_ds[r][c] = ds;
            __syncthreads();
            float dr[KB];
#pragma unroll
            for (int cc = 0; cc < KB; ++cc) {
                dr[cc] = s_ds[r][cc];
            }
#pragma unroll
            for (int j = 0; j < kCols; ++j) {
                const int col = c + 16 * j;
                if (col < a.d_qk) {
                    float t = dq[j];
#pragma unroll
                    for (int cc = 0; cc < KB; ++cc) {
                        t += dr[cc] * s_k[cc * kStride + col];
                    }
                    dq[j] = t;
                }
            }
        }
        if (row_in) {
#pragma unroll
            for (int j = 0; j < kCols; ++j) {
                const int col = c + 16 * j;
                if (col < a.d_qk) {
                    dq_out[(si.q0 + row) * q_row_elems + static_cast<int64_t>(h) * a.d_qk + col] = static_cast<T>(dq[j]);
                }
            }
        }
    }
}

template <typename T, int MAXD>
__global__ __launch_bounds__(256) void hstu_bwd_generic_dkv_kernel(const BwdArgs a)
{
    constexpr int RB = kGenericBwdRows, KB = kGenericBwdRows, kStride = MAXD + 4, kCols = MAXD / 16;
    __shared__ __attribute__((aligned(16))) float s_q[RB * kStride];
    __shared__ __attribute__((aligned(16))) float s_g[RB * kStride];
    __shared__ __attribute__((aligned(16))) float s_k[KB * kStride];
    __shared__ __attribute__((aligned(16))) float s_v[KB * kStride];
    __shared__ float s_p[KB][RB + 1];
    __shared__ float s_ds[KB][RB + 1];

    const int tid = threadIdx.x;
    const int per_level = a.n_batch * a.n_heads_k;
    const int kt_idx = blockIdx.x / per_level;
    const int rem = blockIdx.x - kt_idx * per_level;
    const int b = rem / a.n_heads_k;
    const int hk = rem - b * a.n_heads_k;
    const SeqInfo si = load_seq(a, b);
    const int sq = si.sq, sk = si.sk;
    const int c0 = kt_idx * kBlockM;
    if (c0 >= sk) {
        return;
    }
    const int64_t q_row_elems = static_cast<int64_t>(a.n_heads_q) * a.d_qk;
    const int64_t g_row_elems = static_cast<int64_t>(a.n_heads_q) * a.d_v;
    const int64_t k_row_elems = static_cast<int64_t>(a.n_heads_k) * a.d_qk;
    const int64_t v_row_elems = static_cast<int64_t>(a.n_heads_k) * a.d_v;
    const int kr = tid >> 4, c = tid & 15;
    const int d_qk4 = (a.d_qk + 3) & ~3;
    T* const dk_out = static_cast<T*>(a.dk);
    T* const dv_out = static_cast<T*>(a.dv);

    for (int pass = 0; pass < kBlockM / KB; ++pass) {
        const int kb = c0 + pass * KB;
        if (kb >= sk) {
            break;  // (the same for every thread)
        }
        const int key = kb + kr;
        const bool key_in = key < sk;
        __syncthreads();  // the previous pass is done with s_k / s_v
        generic_stage_rows<T>(s_k, kStride, a.k, si.k0, k_row_elems, static_cast<int64_t>(hk) * a.d_qk, kb, sk, a.d_qk, d_qk4, tid);
        generic_stage_rows<T>(s_v, kStride, a.v, si.k0, v_row_elems, static_cast<int64_t>(hk) * a.d_v, kb, sk, a.d_v, a.d_v, tid);
        float dk[kCols], dv[kCols];
#pragma unroll
        for (int j = 0; j < kCols; ++j) {
            dk[j] = 0.0f;
            dv[j] = 0.0f;
        }
        // the first query row that can see a key of this pass: key j is hidden from row i when j > i + delta, unless
        // row i is a context row and j lies in the history
        int row_first = 0;
        if (a.mask_type == 0 && !(si.n_ctx > 0 && kb < si.hist_k)) {
            const int first = kb - si.delta;
            row_first = first > 0 ? (first / RB) * RB : 0;
        }
        for (int hq = hk * a.head_ratio; hq < (hk + 1) * a.head_ratio; ++hq) {
            const int64_t bias_plane = (static_cast<int64_t>(b) * a.n_heads_q + hq) * a.max_q * static_cast<int64_t>(a.max_k);
            for (int rb = row_first; rb < sq; rb += RB) {
                __syncthreads();  // the previous tile's products are done (and s_k / s_v are written)
                generic_stage_rows<T>(s_q, kStride, a.q, si.q0, q_row_elems, static_cast<int64_t>(hq) * a.d_qk, rb, sq, a.d_qk, d_qk4, tid);
                generic_stage_rows<T>(s_g, kStride, a.grad, si.q0, g_row_elems, static_cast<int64_t>(hq) * a.d_v, rb, sq, a.d_v, a.d_v, tid);
                __syncthreads();
                const int row = rb + c;
                float p = 0.0f, ds = 0.0f;
                if (key_in && row < sq) {
                    int lim, hole_lo, hole_hi;
                    row_bounds(si, a.mask_type, a.target_group, row, lim, hole_lo, hole_hi);
                    if (key < lim && !(key >= hole_lo && key < hole_hi)) {
                        float s = generic_dot(s_q + c * kStride, s_k + kr * kStride, d_qk4 / 4);
                        const float dp = generic_dot(s_g + c * kStride, s_v + kr * kStride, a.d_v / 4);
                        const int64_t at = bias_plane + static_cast<int64_t>(row) * a.max_k + key;
                        if (a.rab != nullptr) {
                            s += generic_load<T>(a.rab, at);
                        }
                        const float x = s * a.alpha;
                        const float sig = 1.0f / (1.0f + __expf(-x));
                        const float m = a.mask_type == 3 ? generic_load<T>(a.mask, at) : 1.0f;
                        p = x * sig * a.scale * m;
                        ds = a.alpha * a.scale * m * dp * sig * (1.0f + x * (1.0f - sig));
                    }
                }
                s_p[kr][c] = p;
                s_ds[kr][c] = ds;
                __syncthreads();
                float pr[RB], dr[RB];
#pragma unroll
                for (int cc = 0; cc < RB; ++cc) {
                    pr[cc] = s_p[kr][cc];
                    dr[cc] = s_ds[kr][cc];
                }
#pragma unroll
                for (int j = 0; j < kCols; ++j) {
                    const int col = c + 16 * j;
                    if (col < a.d_v) {
                        float t = dv[j];
#pragma unroll
                        for (int cc = 0; cc < RB; ++cc) {
                            t += pr[cc] * s_g[cc * kStride + col];
                        }
                        dv[j] = t;
                    }
                    if (col < a.d_qk) {
                        float t = dk[j];
#pragma unroll
                        for (int cc = 0; cc < RB; ++cc) {
                            t += dr[cc] * s_q[cc * kStride + col];
                        }
                        dk[j] = t;
                    }
                }
            }
        }
        if (key_in) {
#pragma unroll
            for (int j = 0; j < kCols; ++j) {
                const int col = c + 16 * j;
                if (col < a.d_qk) {
                    dk_out[(si.k0 + key) * k_row_elems + static_cast<int64_t>(hk) * a.d_qk + col] = static_cast<T>(dk[j]);
                }
                if (col < a.d_v) {
                    dv_out[(si.k0 + key) * v_row_elems + static_cast<int64_t>(hk) * a.d_v + col] = static_cast<T>(dv[j]);
                }
            }
        }
    }
}

}  // namespace hstu
