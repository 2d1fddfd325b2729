// Zero-fill of a byte range shared out over the workgroups of a launch, for kernels that clear an output beside
// their own work (the key-tile kernel of the backward clears the attn_bias gradient, which the query-tile kernel
// launched after it then writes where its tiles sweep: the clear costs that compute-bound kernel nothing measurable,
// where a fill of its own took 68 us for 537 MB ahead of a 430 us backward).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hstu {

// Workgroup `wg` of `n_wgs` (each `threads` wide, this thread `t`) clears its share of bytes [0, n_bytes) at `p`
// (2-byte aligned, n_bytes even): 16-byte non-temporal stores, consecutive lanes on consecutive pieces, over the
// 16-byte aligned body; the first workgroup takes the few bytes ahead of it and the last one those behind it.
__device__ __forceinline__ void clear_share(void* p, int64_t n_bytes, unsigned wg, unsigned n_wgs, int t, int threads)
{
    typedef uint32_t piece_t __attribute__((ext_vector_type(4)));
    uint8_t* const base = static_cast<uint8_t*>(p);
    int64_t head = static_cast<int64_t>((16u - (reinterpret_cast<uintptr_t>(base) & 15u)) & 15u);
    head = head < n_bytes ? head : n_bytes;
    const int64_t pieces = (n_bytes - head) / 16;
    const int64_t tail_at = head + pieces * 16;
    if (wg == 0) {
        for (int64_t e = 2 * static_cast<int64_t>(t); e < head; e += 2 * static_cast<int64_t>(threads)) {
            *reinterpret_cast<uint16_t*>(base + e) = 0;
        }
    }
    if (wg == n_wgs - 1) {
        for (int64_t e = tail_at + 2 * static_cast<int64_t>(t); e < n_bytes; e += 2 * static_cast<int64_t>(threads)) {
            *reinterpret_cast<uint16_t*>(base + e) = 0;
        }
    }
    const int64_t per = (pieces + n_wgs - 1) / n_wgs;
    const int64_t first = static_cast<int64_t>(wg) * per;
    const int64_t last = first + per < pieces ? first + per : pieces;
    piece_t* const body = reinterpret_cast<piece_t*>(base + head);
    const piece_t zero = {0u, 0u, 0u, 0u};
    for (int64_t i = first + t; i < last; i += threads) {
        __builtin_nontemporal_store(zero, body + i);
    }
}

}  // namespace hstu
