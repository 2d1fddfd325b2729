// Paged K/V for the HSTU forward on gfx950 (MI355X): the key / value rows of a sequence are its cached history,
// kept in fixed-size pages of a cache tensor [num_pages, 2, page_size, heads_k, dim] and named by a page table,
// followed by the rows of its new target tokens, which arrive in the k / v inputs
// (ascendc/attention/hstu_v1/hstu_forward_v1/op_kernel/atlas950/hstu_paged_forward_kernel.h, FetchKvMayFromCache;
//  golden: hstu_forward_v1/test/pytest/test_hstu_paged.py:213-262, common.py:255-300).
//
// This kernel lays those rows out contiguously, [seq_offset_k[b], seq_offset_k[b + 1]) per sequence, in a workspace;
// the jagged forward kernel then runs on the workspace as on any K / V ("delta" form, grouped targets).  One
// workgroup per key row; K and V rows are copied 16 bytes per lane.  HBM-bound: every K / V byte is read and written
// once here on top of what the forward reads.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hstu_fwd_kernel.hip.h"

namespace hstu {



__global__ __launch_bounds__(kGatherThreads) void hstu_paged_gather_kernel(const PagedGatherArgs a)
{
    const int64_t row = blockIdx.x;  // key row in the gathered layout
    // the sequence that owns the row: last b with offs_k[b] <= row (empty sequences are skipped by taking the last)
    int lo = 0, hi = a.n_batch;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (load_index_uniform(a.offs_k, mid, a.idx64) <= row) {
            lo = mid;
        } else {
            hi = mid;
        }
    }
    const int b = lo;
    const int64_t k0 = load_index_uniform(a.offs_k, b, a.idx64);
    const int64_t k1 = load_index_uniform(a.offs_k, b + 1, a.idx64);
    const uint8_t* src_k = nullptr;  // null: the row belongs to no sequence or its source is out of range -> zeros
    const uint8_t* src_v = nullptr;
    if (row >= k0 && row < k1) {
        const int64_t q0 = load_index_uniform(a.offs_q, b, a.idx64);
        const int64_t q1 = load_index_uniform(a.offs_q, b + 1, a.idx64);
        int64_t n_tgt = a.num_tgt ? load_index_uniform(a.num_tgt, b, a.idx64) : 0;
        const int64_t sk = k1 - k0;
        n_tgt = n_tgt < 0 ? 0 : (n_tgt > sk ? sk : n_tgt);
        const int64_t n_cached = sk - n_tgt;
        const int64_t r = row - k0;
        if (r < n_cached) {
            const int64_t p0 = load_index_uniform(a.page_offsets, b, a.idx64);
            const int64_t p1 = load_index_uniform(a.page_offsets, b + 1, a.idx64);
            const int64_t p = p0 + r / a.page_size;
            if (p >= 0 && p < p1 && p < a.n_page_ids) {
                const int64_t pid = load_index_uniform(a.page_ids, p, a.idx64);
                if (pid >= 0 && pid < a.num_pages) {
                    const int64_t in_page = r % a.page_size;
                    const uint8_t* page = static_cast<const uint8_t*>(a.kv_cache) + pid * 2 * a.page_size * static_cast<int64_t>(a.row_bytes);
                    src_k = page + in_page * a.row_bytes;
                    src_v = page + (a.page_size + in_page) * static_cast<int64_t>(a.row_bytes);
                }
            }
        } else {
            // target row j of the sequence: the j-th of the last n_tgt rows of its segment of the inputs
            const int64_t t = q1 - n_tgt + (r - n_cached);
            if (t >= q0 && t < q1 && t < a.total_q) {
                src_k = static_cast<const uint8_t*>(a.k) + t * a.row_bytes;
                src_v = static_cast<const uint8_t*>(a.v) + t * a.row_bytes;
            }
        }
    }
    typedef __attribute__((ext_vector_type(4))) uint32_t u4;
    uint8_t* const dst_k = static_cast<uint8_t*>(a.k_out) + row * a.row_bytes;
    uint8_t* const dst_v = static_cast<uint8_t*>(a.v_out) + row * a.row_bytes;
    const u4 zero = {0u, 0u, 0u, 0u};
    for (int off = threadIdx.x * 16; off < a.row_bytes; off += kGatherThreads * 16) {
        *reinterpret_cast<u4*>(dst_k + off) = src_k ? *reinterpret_cast<const u4*>(src_k + off) : zero;
        *reinterpret_cast<u4*>(dst_v + off) = src_v ? *reinterpret_cast<const u4*>(src_v + off) : zero;
    }
}

}  // namespace hstu
