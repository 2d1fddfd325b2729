// LayerNorm(x) * u over the rows of a [rows, cols] matrix, gfx950.
//
//   mean = sum(x) / cols;  var = sum((x - mean)^2) / cols;  rstd = 1 / sqrt(var + eps)
//   out  = ((x - mean) * rstd * gamma + beta) * u
//
// (two-pass variance and this order of operations as in the reference kernel,
//  ascendc/activation/ln_mul/op_kernel/ln_mul_kernel.h:238-277).  One refinement: the fp32 sum of a long row with a
// large common offset leaves the first mean off by a few units in its last place, which the reference carries into
// every centred value; here the sum of the centred values (zero for an exact mean) is reduced beside the sum of their
// squares and mean and variance are corrected by it, which costs one more cross-lane reduction and no memory traffic.
//
// The operation moves 3 values per element (x, u in; out) and does a dozen flops on them: HBM-bound.  A row is owned
// by a group of G lanes (8..64 lanes of one wavefront, or all 256 lanes of a workgroup), sized so that the row fits
// the group's registers as NV 16-byte chunks per lane: x and u are read once, with every load of the row in flight
// before the first use, the two reductions run on registers (cross-lane moves; through LDS only for G = 256) and the
// result is written once.  Rows that cannot be cut into aligned 16-byte chunks, or that are longer than 256 lanes can
// hold, take the element-wise form of the same kernel (VEC = false), which re-reads the row for the second and third
// pass; those reads hit in the cache, the row having just been streamed by the same lanes.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hstu_args.h"

namespace hstu {

typedef uint32_t ln_chunk_t __attribute__((ext_vector_type(4)));  // 16 bytes of a row
typedef float ln_f32x4_t __attribute__((ext_vector_type(4)));

struct ln_f32_tag {};
struct ln_bf16_tag {};
struct ln_f16_tag {};

template <typename Tag>
struct ln_traits;
template <>
struct ln_traits<ln_f32_tag> {
    using elem_t = float;
    static constexpr int kPerChunk = 4;
    static __device__ __forceinline__ float load(const void* p, int64_t i) { return static_cast<const float*>(p)[i]; }
    static __device__ __forceinline__ void store(void* p, int64_t i, float v) { static_cast<float*>(p)[i] = v; }
    static __device__ __forceinline__ void unpack(const ln_chunk_t& c, float* f)
    {
        const ln_f32x4_t v = __builtin_bit_cast(ln_f32x4_t, c);
        f[0] = v[0];
        f[1] = v[1];
        f[2] = v[2];
        f[3] = v[3];
    }
    static __device__ __forceinline__ ln_chunk_t pack(const float* f)
    {
        // the four floats are cast as one vector: this compiler turns four scalar casts inside a vector
        // initialiser into four copies of the first
        const ln_f32x4_t v = {f[0], f[1], f[2], f[3]};
        return __builtin_bit_cast(ln_chunk_t, v);
    }
};
template <>
struct ln_traits<ln_bf16_tag> {
    using elem_t = __bf16;
    static constexpr int kPerChunk = 8;
    static __device__ __forceinline__ float load(const void* p, int64_t i)
    {
        return static_cast<float>(static_cast<const __bf16*>(p)[i]);
    }
    static __device__ __forceinline__ void store(void* p, int64_t i, float v)
    {
        static_cast<__bf16*>(p)[i] = static_cast<__bf16>(v);  // round to nearest even
    }
    static __device__ __forceinline__ void unpack(const ln_chunk_t& c, float* f)
    {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w = c[i];
            f[2 * i] = __builtin_bit_cast(float, w << 16);
            f[2 * i + 1] = __builtin_bit_cast(float, w & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ ln_chunk_t pack(const float* f)
    {
        typedef __attribute__((ext_vector_type(8))) __bf16 octet_t;
        octet_t r;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            r[i] = static_cast<__bf16>(f[i]);
        }
        return __builtin_bit_cast(ln_chunk_t, r);
    }
};
template <>
struct ln_traits<ln_f16_tag> {
    using elem_t = _Float16;
    static constexpr int kPerChunk = 8;
    static __device__ __forceinline__ float load(const void* p, int64_t i)
    {
        return static_cast<float>(static_cast<const _Float16*>(p)[i]);
    }
    static __device__ __forceinline__ void store(void* p, int64_t i, float v)
    {
        static_cast<_Float16*>(p)[i] = static_cast<_Float16>(v);
    }
    static __device__ __forceinline__ void unpack(const ln_chunk_t& c, float* f)
    {
        typedef __attribute__((ext_vector_type(8))) _Float16 octet_t;
        const octet_t r = __builtin_bit_cast(octet_t, c);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            f[i] = static_cast<float>(r[i]);
        }
    }
    static __device__ __forceinline__ ln_chunk_t pack(const float* f)
    {
        typedef __attribute__((ext_vector_type(8))) _Float16 octet_t;
        octet_t r;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            r[i] = static_cast<_Float16>(f[i]);
        }
        return __builtin_bit_cast(ln_chunk_t, r);
    }
};

// sum over the G lanes that own a row; every lane of the group gets the total.  G <= 64: the group is an aligned
// slice of one wavefront.  G = 256: the workgroup, through four partial sums in LDS (each reduction of a row has a
// `slot` of its own, so that none overwrites partials another wavefront still reads).
template <int G>
__device__ __forceinline__ float group_sum(float v, float* s_part, int slot)
{
    constexpr int kWave = G < 64 ? G : 64;
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        v += __shfl_xor(v, off, 64);
    }
    if constexpr (G == 256) {
        if ((threadIdx.x & 63) == 0) {
            s_part[slot * 4 + (threadIdx.x >> 6)] = v;
        }
        __syncthreads();
        v = (s_part[slot * 4] + s_part[slot * 4 + 1]) + (s_part[slot * 4 + 2] + s_part[slot * 4 + 3]);
    }
    return v;
}

// gamma / beta are fp32 or of the element type of x
template <typename Tag>
__device__ __forceinline__ float load_affine(const void* p, int64_t i, bool is_f32)
{
    return is_f32 ? static_cast<const float*>(p)[i] : ln_traits<Tag>::load(p, i);
}

template <typename Tag>
__device__ __forceinline__ void load_affine_chunk(const void* p, int64_t first, bool is_f32, float* f)
{
    using T = ln_traits<Tag>;
    if (is_f32) {
        const ln_chunk_t* q = reinterpret_cast<const ln_chunk_t*>(static_cast<const float*>(p) + first);
#pragma unroll
        for (int j = 0; j < T::kPerChunk / 4; ++j) {
            ln_traits<ln_f32_tag>::unpack(q[j], f + 4 * j);
        }
    } else {
        const ln_chunk_t c = *reinterpret_cast<const ln_chunk_t*>(static_cast<const typename T::elem_t*>(p) + first);
        T::unpack(c, f);
    }
}

template <typename Tag, int G, int NV, bool VEC>
__global__ __launch_bounds__(kLnMulThreads) void ln_mul_kernel(const LnMulArgs a)
{
    using T = ln_traits<Tag>;
    constexpr int EPC = T::kPerChunk;
    __shared__ float s_part[12];
    const int64_t row = (static_cast<int64_t>(blockIdx.x) * kLnMulThreads + threadIdx.x) / G;
    const int lane = threadIdx.x % G;
    // a group past the last row has nothing to do (G = 256: one row per workgroup and one workgroup per row, so the
    // lanes that share the barriers of group_sum stay or leave together)
    if (row >= a.rows) {
        return;
    }
    const int64_t base = row * a.cols;
    const float inv_n = 1.0f / static_cast<float>(a.cols);
    const bool affine_f32 = a.affine_f32 != 0;

    if constexpr (VEC) {
        const typename T::elem_t* xr = static_cast<const typename T::elem_t*>(a.x) + base;
        const typename T::elem_t* ur = static_cast<const typename T::elem_t*>(a.u) + base;
        typename T::elem_t* outr = static_cast<typename T::elem_t*>(a.out) + base;
        const int n_chunks = static_cast<int>(a.cols / EPC);
        // every lane loads NV chunks without a branch (a chunk index past the row is clamped to the last chunk and its
        // values are replaced by zeros below), so that all loads of the row are in flight at once
        ln_chunk_t xc[NV], uc[NV];
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = min(lane + i * G, n_chunks - 1);
            xc[i] = __builtin_nontemporal_load(reinterpret_cast<const ln_chunk_t*>(xr) + c);
            uc[i] = __builtin_nontemporal_load(reinterpret_cast<const ln_chunk_t*>(ur) + c);
        }
        float xf[NV][EPC];
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            T::unpack(xc[i], xf[i]);
            const bool valid = lane + i * G < n_chunks;
#pragma unroll
            for (int j = 0; j < EPC; ++j) {
                sum += valid ? xf[i][j] : 0.0f;
            }
        }
        const float mean = group_sum<G>(sum, s_part, 0) * inv_n;
        float sq = 0.0f, rest = 0.0f;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const bool valid = lane + i * G < n_chunks;
#pragma unroll
            for (int j = 0; j < EPC; ++j) {
                xf[i][j] = valid ? xf[i][j] - mean : 0.0f;
                rest += xf[i][j];
                sq += xf[i][j] * xf[i][j];
            }
        }
        const float shift = group_sum<G>(rest, s_part, 1) * inv_n;
        const float var = fmaxf(group_sum<G>(sq, s_part, 2) * inv_n - shift * shift, 0.0f);
        const float rstd = 1.0f / sqrtf(var + a.epsilon);
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = lane + i * G;
            const int cc = min(c, n_chunks - 1);
            float g[EPC], b[EPC], uf[EPC], y[EPC];
            load_affine_chunk<Tag>(a.gamma, static_cast<int64_t>(cc) * EPC, affine_f32, g);
            load_affine_chunk<Tag>(a.beta, static_cast<int64_t>(cc) * EPC, affine_f32, b);
            T::unpack(uc[i], uf);
#pragma unroll
            for (int j = 0; j < EPC; ++j) {
                y[j] = (((xf[i][j] - shift) * rstd) * g[j] + b[j]) * uf[j];
            }
            if (c < n_chunks) {
                __builtin_nontemporal_store(T::pack(y), reinterpret_cast<ln_chunk_t*>(outr) + c);
            }
        }
    } else {
        const int64_t n = a.cols;
        float sum = 0.0f;
        for (int64_t j = lane; j < n; j += G) {
            sum += T::load(a.x, base + j);
        }
        const float mean = group_sum<G>(sum, s_part, 0) * inv_n;
        float sq = 0.0f, rest = 0.0f;
        for (int64_t j = lane; j < n; j += G) {
            const float d = T::load(a.x, base + j) - mean;
            rest += d;
            sq += d * d;
        }
        const float shift = group_sum<G>(rest, s_part, 1) * inv_n;
        const float var = fmaxf(group_sum<G>(sq, s_part, 2) * inv_n - shift * shift, 0.0f);
        const float rstd = 1.0f / sqrtf(var + a.epsilon);
        for (int64_t j = lane; j < n; j += G) {
            const float d = T::load(a.x, base + j) - mean - shift;
            const float y = ((d * rstd) * load_affine<Tag>(a.gamma, j, affine_f32) + load_affine<Tag>(a.beta, j, affine_f32)) *
                            T::load(a.u, base + j);
            T::store(a.out, base + j, y);
        }
    }
}

}  // namespace hstu
