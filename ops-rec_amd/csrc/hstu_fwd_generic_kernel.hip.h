// HSTU jagged attention forward for gfx950: the shapes the tuned kernels do not take.
//
// The reference accepts any q/k head dim in [1, 512] and any v head dim in [16, 512] in steps of 16
// (ascendc/attention/hstu_v1/hstu_forward_v1/op_host/tiling_policy.cpp:68-93).  The MFMA kernels of this library
// are built for head dims up to 256 with a q/k head dim that is a multiple of 8 (16-byte chunks).  This kernel
// covers the rest -- head dims up to 512, any q/k head dim, bf16 / fp16 / fp32 / fp8-e4m3 -- so that every input the reference
// takes runs here too.  It is written for coverage, not for speed: plain fp32 arithmetic on the vector unit, the
// same semantics (O = (silu(alpha (Q K^T + rab)) * silu_scale * M) V, masks, grouped heads, longer key sequences)
// restated without any of the tuned kernels' machinery, one workgroup per 128-row query tile as in
// hstu_fwd_f32_kernel so that the host launches both the same way.
//
// A workgroup walks its 128 rows 16 at a time.  For 16 rows and 16 keys, thread (r, c) of the 256 computes the
// score of row r and key c from fp32 copies of the Q and K rows in LDS (zero-padded to a multiple of 4 floats and
// read 16 bytes at a time; row stride padded by 4 floats so that the 16 key rows read together fall into different
// banks), applies bias, SiLU, scale and visibility, and leaves P in LDS; thread (r, c) then owns the output columns
// 4c .. 4c + 3, 4c + 64 .. of row r and adds P[r, :] . V[:, columns].  Scores are not rounded to the input type before the second product.
#pragma once
#include "hstu_fwd_kernel.hip.h"

namespace hstu {

constexpr int kGenericMaxDim = 512;

// fp8-e4m3 (OCP e4m3fn) elements, for the head dims the tuned fp8 kernels do not take (above 256, or a q/k head dim
// that is not a multiple of 16).  Q, K, V, attn_bias and the custom mask are e4m3; the score is brought to its real
// scale with the per-head dequantisation scales, P is rounded to e4m3 (nearest even, saturating at +-448) before or
// after silu_scale is applied (FwdArgs::fp8_scaled_p, as in the tuned kernels), the second product and its sum are
// fp32, and the V scale (and silu_scale in the second case) goes on the fp32 output, which is OutT (fp16 or bf16).
struct f8e4m3_elem {
    uint8_t bits;
};

template <typename T>
__device__ __forceinline__ float generic_load(const void* p, int64_t i)
{
    return static_cast<float>(static_cast<const T*>(p)[i]);
}
template <>
__device__ __forceinline__ float generic_load<f8e4m3_elem>(const void* p, int64_t i)
{
    return __builtin_amdgcn_cvt_f32_fp8(static_cast<int>(static_cast<const uint8_t*>(p)[i]), 0);
}
// x rounded to e4m3 and back
__device__ __forceinline__ float round_to_e4m3(float x)
{
    x = x > 448.0f ? 448.0f : (x < -448.0f ? -448.0f : x);  // (a NaN passes through)
    const int packed = __builtin_amdgcn_cvt_pk_fp8_f32(x, 0.0f, 0, false);
    return __builtin_amdgcn_cvt_f32_fp8(packed, 0);
}

template <typename T, typename OutT = T>
__global__ __launch_bounds__(256) void hstu_fwd_generic_kernel(const FwdArgs a)
{
    constexpr bool F8 = std::is_same<T, f8e4m3_elem>::value;
    constexpr int kThreads = 256;
    constexpr int RB = 16;  // query rows per pass
    constexpr int KB = 16;  // keys per tile
    constexpr int kStride = kGenericMaxDim + 4;  // floats per staged Q / K row: 16-byte reads, rows 4 banks apart
    __shared__ __attribute__((aligned(16))) float s_q[RB * kStride];
    __shared__ __attribute__((aligned(16))) float s_k[KB * kStride];
    __shared__ __attribute__((aligned(16))) float s_v[KB * kGenericMaxDim];
    __shared__ float s_p[RB][KB + 1];

    const int tid = threadIdx.x;
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
    q1 = q1 < a.total_q ? q1 : a.total_q;
    k1 = k1 < a.total_k ? k1 : a.total_k;
    q0 = q0 < 0 ? 0 : q0;
    k0 = k0 < 0 ? 0 : k0;
    int sq = static_cast<int>(q1 > q0 ? q1 - q0 : 0);
    int sk = static_cast<int>(k1 > k0 ? k1 - k0 : 0);
    sq = sq < a.max_q ? sq : a.max_q;
    sk = sk < a.max_k ? sk : a.max_k;

    OutT* const out = static_cast<OutT*>(a.out);
    const int64_t o_row_elems = static_cast<int64_t>(a.n_heads_q) * a.d_v;
    if (qt == 0) {  // rows past the last offset belong to no sequence: zero-fill them
        const int64_t last = load_index(a.offs_q, a.n_batch, a.idx64);
        const int64_t first_tail = last < 0 ? 0 : last;
        const int64_t n_tail = (a.total_q > first_tail ? a.total_q - first_tail : 0) * o_row_elems;
        OutT* tail = out + first_tail * o_row_elems;
        for (int64_t e = static_cast<int64_t>(bhid) * kThreads + tid; e < n_tail; e += static_cast<int64_t>(a.bh) * kThreads) {
            tail[e] = static_cast<OutT>(0.0f);
        }
    }
    const int r0 = qt * kBlockM;
    if (r0 >= sq) {
        return;
    }
    int n_ctx = 0, n_tgt = 0;
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
    const int hist_k = sk - n_tgt;
    const int64_t q_row_elems = static_cast<int64_t>(a.n_heads_q) * a.d_qk;
    const int64_t k_row_elems = static_cast<int64_t>(a.n_heads_k) * a.d_qk;
    const int64_t v_row_elems = static_cast<int64_t>(a.n_heads_k) * a.d_v;
    const int64_t bias_plane = (static_cast<int64_t>(b) * a.n_heads_q + h) * a.max_q * static_cast<int64_t>(a.max_k);
    // fp8: raw score -> real score, what P is multiplied by before it is rounded, what the fp32 output is multiplied by
    float score_scale = 1.0f, p_scale = a.silu_scale, out_scale = 1.0f;
    if constexpr (F8) {
        const float qs = a.q_descale ? a.q_descale[h] : 1.0f;
        const float ks = a.k_descale ? a.k_descale[hk] : 1.0f;
        const float vs = a.v_descale ? a.v_descale[hk] : 1.0f;
        score_scale = qs * ks;
        p_scale = a.fp8_scaled_p ? a.silu_scale : 1.0f;
        out_scale = (a.fp8_scaled_p ? 1.0f : a.silu_scale) * vs;
    }
    const int r = tid >> 4, c = tid & 15;
    constexpr int kMaxCols = kGenericMaxDim / 64;  // groups of 4 consecutive output columns per thread
    const int d_qk4 = (a.d_qk + 3) & ~3;                 // Q / K rows are staged zero-padded to a multiple of 4
    typedef __attribute__((ext_vector_type(4))) float f32x4_t;

    for (int pass = 0; pass < kBlockM / RB; ++pass) {
        const int rb = r0 + pass * RB;
        if (rb >= sq) {
            break;  // (the same for every thread)
        }
        const int row = rb + r;
        const bool row_in = row < sq;
        // visibility of key j from this row: j < lim and not in [hole_lo, hole_hi)
        // (ascendc/attention/hstu_v1/hstu_forward_v1/op_kernel/atlas950/hstu_dense_causal_mask.h:186-260)
        int lim = sk, hole_lo = 0, hole_hi = 0;
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
        }
        // keys any of the 16 rows can see
        int kmax = sk;
        if (a.mask_type == 0) {
            const int last_row = (rb + RB < sq ? rb + RB : sq) - 1;
            kmax = last_row + delta + 1;
            if (rb < n_ctx) {
                kmax = kmax > hist_k ? kmax : hist_k;
            }
            kmax = kmax < 0 ? 0 : (kmax > sk ? sk : kmax);
        }
        __syncthreads();  // the previous pass is done with s_q
        for (int e = tid; e < RB * d_qk4; e += kThreads) {
            const int rr = e / d_qk4, dd = e - rr * d_qk4;
            const int qrow = rb + rr;
            s_q[rr * kStride + dd] = (qrow < sq && dd < a.d_qk) ? generic_load<T>(a.q, (q0 + qrow) * q_row_elems + static_cast<int64_t>(h) * a.d_qk + dd) : 0.0f;
        }
        f32x4_t acc[kMaxCols];
#pragma unroll
        for (int jj = 0; jj < kMaxCols; ++jj) {
            acc[jj] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        }
        for (int kt = 0; kt * KB < kmax; ++kt) {
            const int key0 = kt * KB;
            __syncthreads();  // the previous tile's products are done (and s_q is written)
            for (int e = tid; e < KB * d_qk4; e += kThreads) {
                const int kr = e / d_qk4, dd = e - kr * d_qk4;
                const int key = key0 + kr;
                s_k[kr * kStride + dd] = (key < sk && dd < a.d_qk) ? generic_load<T>(a.k, (k0 + key) * k_row_elems + static_cast<int64_t>(hk) * a.d_qk + dd) : 0.0f;
            }
            for (int e = tid; e < KB * a.d_v; e += kThreads) {
                const int kr = e / a.d_v, dd = e - kr * a.d_v;
                const int key = key0 + kr;
                s_v[kr * kGenericMaxDim + dd] = key < sk ? generic_load<T>(a.v, (k0 + key) * v_row_elems + static_cast<int64_t>(hk) * a.d_v + dd) : 0.0f;
            }
            __syncthreads();
            const int key = key0 + c;
            float p = 0.0f;
            if (row_in && key < lim && !(key >= hole_lo && key < hole_hi)) {
                const f32x4_t* qr = reinterpret_cast<const f32x4_t*>(s_q + r * kStride);
                const f32x4_t* kr = reinterpret_cast<const f32x4_t*>(s_k + c * kStride);
                f32x4_t s4 = {0.0f, 0.0f, 0.0f, 0.0f};
                for (int dd = 0; dd < d_qk4 / 4; ++dd) {
                    s4 += qr[dd] * kr[dd];
                }
                float s = ((s4[0] + s4[1]) + (s4[2] + s4[3])) * score_scale;
                const int64_t at = bias_plane + static_cast<int64_t>(row) * a.max_k + key;
                if (a.rab != nullptr) {
                    s += generic_load<T>(a.rab, at);
                }
                const float x = s * a.alpha;
                p = x / (1.0f + __expf(-x)) * p_scale;
                if (a.mask_type == 3) {
                    p *= generic_load<T>(a.mask, at);
                }
                if constexpr (F8) {
                    p = round_to_e4m3(p);
                }
            }
            s_p[r][c] = p;
            __syncthreads();
            float pr[KB];
#pragma unroll
            for (int cc = 0; cc < KB; ++cc) {
                pr[cc] = s_p[r][cc];
            }
#pragma unroll
            for (int jj = 0; jj < kMaxCols; ++jj) {
                const int col = 4 * c + 64 * jj;  // d_v is a multiple of 16: a group of 4 columns is inside or outside
                if (col < a.d_v) {
                    f32x4_t t = acc[jj];
#pragma unroll
                    for (int cc = 0; cc < KB; ++cc) {
                        t += pr[cc] * *reinterpret_cast<const f32x4_t*>(s_v + cc * kGenericMaxDim + col);
                    }
                    acc[jj] = t;
                }
            }
        }
        if (row_in) {
#pragma unroll
            for (int jj = 0; jj < kMaxCols; ++jj) {
                const int col = 4 * c + 64 * jj;
                if (col < a.d_v) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        out[(q0 + row) * o_row_elems + static_cast<int64_t>(h) * a.d_v + col + e] = static_cast<OutT>(acc[jj][e] * out_scale);
                    }
                }
            }
        }
    }
}

}  // namespace hstu
