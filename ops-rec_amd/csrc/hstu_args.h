// Argument blocks of the kernels and the few constants the host side shares with them (no device code here).
#pragma once
#include <stdint.h>

namespace hstu {

constexpr int kBlockM = 128;  // query rows per workgroup
constexpr int kWaveM = 32;    // query rows per wavefront
// workgroups per CU the backward kernels are compiled for (not persistent: the hardware places as many as fit).  At
// the head-dim slot 64 a third one fits where the kernel needs no more than 168 registers: the key-tile kernel
// without bias or custom mask (173 as compiled for two), the query-tile kernel unless it takes both (158 - 167; 180
// with both); 25 - 33 KB of LDS each.  Measured (bf16, B32 H8 d64 L1024): backward 304 -> 267 us.
constexpr int bwd_dkv_wgs_per_cu(int d, bool rab, bool mask) { return (!rab && !mask && d <= 64) ? 3 : (d <= 128 ? 2 : 1); }
// the dK workgroups that read dS back from memory keep neither V nor dO nor the score blocks: 90 / 148 / 137 registers
// and 16 / 32 / 64 KB of LDS at the head-dim slots 64 / 128 / 256
constexpr int bwd_dk_from_ds_wgs_per_cu(int d) { return d <= 64 ? 4 : (d <= 128 ? 3 : 2); }
constexpr int bwd_dq_wgs_per_cu(int d, bool rab, bool mask) { return (!(rab && mask) && d <= 64) ? 3 : (d <= 128 ? 2 : 1); }
// resident workgroups per CU of the forward kernel (registers and LDS): without bias or custom mask four for the
// head-dim slot 32 (127 registers, 25 KB of LDS) and three for 64 (168 registers, 45 KB); three for the slot 32 with
// either a bias or a custom mask (158 / 151 registers); two up to 128, one above
constexpr int fwd_wgs_per_cu(int d, bool rab, bool mask)
{
    return (!rab && !mask && d <= 64) ? (d <= 32 ? 4 : 3) : (d <= 32 && !(rab && mask)) ? 3 : (d <= 128 ? 2 : 1);
}
// Lines per query row of the pair plane in its full form (every 32-key block of the row): odd, so that the 32 lines
// one store instruction of a wavefront writes -- the same block of 32 consecutive rows -- fall on different memory
// channels.  With max_seq_len_k 8192 the plain count, 256 lines = 32 KiB, put them all on one (measured on MI355X, 2
// sequences x 4 heads of 4096 .. 8192 rows: query-tile kernel 445 us, 298 us with the odd pitch).
constexpr int64_t pair_full_pitch_lines(int64_t max_k) { return ((max_k + 31) / 32) | 1; }
constexpr int kShortThreads = 512;  // threads of a workgroup of the forward kernel for short lists (eight wavefronts of 16 query rows)
constexpr int kTinyThreads = 128;   // threads of a workgroup of the backward kernel for tiny sequences (two wavefronts of 16 query rows)
constexpr int kTinyRows = 32;       // the longest sequence (rows and keys) that kernel takes; the forward one: 32 or 64, four threads per row
constexpr int kDqShortThreads = 256;  // threads of a workgroup of the backward's query-tile kernel for short rows (four wavefronts of 16 rows)
constexpr int kDqShortRows = 64;      // query rows of its tile
constexpr int kFewRowsThreads = 256;  // threads of a workgroup of the backward kernel for sequences of few query rows
constexpr int kFewRows = 64;          // the most query rows of a sequence that kernel takes
constexpr int kFwdFewRowsThreads = 512;  // threads of a workgroup of the forward kernel for few query rows (eight wavefronts over row groups and keys)
constexpr int kCounterBlockBytes = 16384;  // head of the workspace: device-side work counters (see the forward kernel)
constexpr int kDkvThreads = 256;   // threads of a workgroup of the key-tile backward kernel
constexpr int kGatherThreads = 128;

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
    int d_qk;        // real head dims (<= the padded template dim)
    int d_v;
    int max_q;
    int max_k;
    int mask_type;
    int target_group;
    int idx64;       // offsets / context / target are int64
    int n_qtiles;    // ceil(max_q / kBlockM)
    int bh;          // n_batch * n_heads_q
    int bias_vec_ok; // rab / mask rows may be read 4 elements (8 bytes) at a time
    int out_vec_ok;  // d_v is a multiple of 8 and `out` is 16-byte aligned: output rows may be written 16 bytes at a time
    float c_exp;     // -alpha * log2(e)
    float c_out;     // alpha * silu_scale
    float alpha;     // fp8 inputs only: the kernel folds the per-head scales in itself
    float silu_scale;
    int fp8_scaled_p;        // fp8 inputs only: 1 = P is multiplied by silu_scale before it is quantised (reference), 0 = after
    const float* q_descale;  // fp8 inputs only; per head, nullptr = 1
    const float* k_descale;
    const float* v_descale;
    unsigned int* counters;  // kCounterBlockBytes at the head of the workspace, cleared ahead of the launch; null for the plain list
    float* ws;           // split variant: room for ws_parts partial outputs of kBlockM x D floats each (may be null)
    uint32_t ws_parts;
    // paged variant: the first (key count - num_target) key rows of a sequence live in pages of kv_cache
    // [num_pages, 2 (K, V), page_size, n_heads_k, d]; k / v then hold the rows of ALL query tokens, of which the last
    // num_target of each sequence are its remaining keys
    const void* kv_cache;
    const void* page_offsets;  // [n_batch + 1]
    const void* page_ids;      // [n_page_ids]
    int64_t num_pages;
    int64_t n_page_ids;
    int page_shift;  // log2(page_size); page_size is 32, 64, 128 or 256
};

struct BwdArgs {
    const void* q;
    const void* k;
    const void* v;
    const void* grad;  // dO
    const void* rab;
    const void* mask;
    void* dq;
    void* dk;
    void* dv;
    void* drab;  // may be null
    void* p_plane;  // where the query-tile kernel leaves dS and P for key-tile workgroups that read them back, or null
    // layout of that plane in the 16-bit kernels (hstu_bwd_kernel.hip.h, pair plane): 128-byte lines per head, and whether
    // the rows of a sequence's 32-row group G hold the blocks 0 .. G only
    int64_t plane_head_lines;
    int plane_tri;
    // Head dims above 256 (hstu_bwd_kernel.hip.h, windows): the kernels of the slot 256 run on halves of the heads.
    // win = 2: q / k / v / grad and the gradients are taken as 2 x heads of half the head dims (n_heads_q, n_heads_k, d_qk
    // and d_v say so), head 2 h + w being window w of head h; planes and the attn_bias tensors are indexed by the real head.
    // win_only >= 0: the launch covers that window only (its grid counts real heads).  Otherwise win = 1, win_only = -1.
    int win;
    int win_only;
    // Order of the (tile level, pair) slots in the grids of the tuned 16-bit kernels (hstu_bwd_kernel.hip.h, slot_of):
    // 0 = level after level (heaviest tiles of all pairs first), 1 = pair after pair, the pairs dealt to the 8 XCDs.
    int pair_major;
    float* partial;  // S and dP summed over the first window, fp32, for the launch that adds the second (or null)
    int64_t drab_clear_bytes;  // > 0: the key-tile kernel clears this many bytes at drab beside its work
    const void* offs_q;
    const void* offs_k;
    const void* num_ctx;
    const void* num_tgt;
    int64_t total_q;
    int64_t total_k;
    int n_batch;
    int n_heads_q;
    int n_heads_k;
    int head_ratio;
    int d_qk;
    int d_v;
    int max_q;
    int max_k;
    int mask_type;
    int target_group;
    int idx64;
    int n_qtiles;     // ceil(max_q / 128)
    int n_ktiles;     // ceil(max_k / 128)
    int bias_vec_ok;  // rab / mask / d rab rows may be accessed 4 elements (8 bytes) at a time (1), 16 bytes (2)
    int grad_vec_ok;  // dq / dk / dv are 16-byte aligned and both head dims multiples of 8: rows may be written 16 bytes at a time
    float alpha;
    float scale;  // silu_scale, resolved
};

struct PagedGatherArgs {
    const void* k;         // [total_q, heads_k, dim]: rows of all tokens; only the target rows are used
    const void* v;
    const void* kv_cache;  // [num_pages, 2, page_size, heads_k, dim]
    void* k_out;           // [total_k, heads_k, dim]
    void* v_out;
    const void* offs_q;    // [n_batch + 1]
    const void* offs_k;    // [n_batch + 1]
    const void* page_offsets;  // [n_batch + 1]
    const void* page_ids;      // [page_offsets[n_batch]]
    const void* num_tgt;       // [n_batch]
    int64_t total_q;
    int64_t total_k;
    int64_t num_pages;
    int64_t n_page_ids;
    int n_batch;
    int page_size;
    int row_bytes;  // heads_k * dim * element size, a multiple of 16
    int idx64;
};

// LayerNorm(x) * u over rows (ln_mul_kernel.hip.h)
constexpr int kLnMulThreads = 256;

struct LnMulArgs {
    const void* x;      // [rows, cols]
    const void* u;      // [rows, cols]
    const void* gamma;  // [cols], fp32 or the element type of x
    const void* beta;   // [cols], like gamma
    void* out;          // [rows, cols]
    int64_t rows;
    int64_t cols;
    float epsilon;
    int affine_f32;  // 1: gamma / beta are fp32; 0: they have the element type of x
};

// in_linear_silu forward (in_linear_silu_kernel.hip.h)
struct InLinearSiluArgs {
    const void* x;       // [m, k], 16-bit
    const void* weight;  // [n, k], 16-bit
    const float* bias;   // [n] or nullptr
    void* user;          // [m, split_end[0]]
    void* value;         // [m, split_end[1] - split_end[0]]
    void* query;         // [m, split_end[2] - split_end[1]]
    void* key;           // [m, n - split_end[2]]
    void* linear_output; // [m, n]
    int64_t m;
    int n;
    int k;
    int split_end[3];  // first column after the user, value and query parts
    int xcd_groups;    // 1: tiles dealt so that all n tiles of an m tile run on one XCD (grid padded to 8 m tiles)
};

// element-wise stage of in_linear_silu's backward (in_linear_silu_bwd_kernel.hip.h)
struct InLinearSiluBwdArgs {
    const void* linear_output;  // [m, n], 16-bit
    const void* user_grad;      // [m, split_end[0]]
    const void* value_grad;     // [m, split_end[1] - split_end[0]]
    const void* query_grad;     // [m, split_end[2] - split_end[1]]
    const void* key_grad;       // [m, n - split_end[2]]
    void* d_mixed;              // [m, n], 16-bit
    float* partial_sums;        // [ceil(m / 64), n] column sums per workgroup row, or nullptr when no bias gradient is wanted
    int64_t m;
    int n;
    int split_end[3];
};

}  // namespace hstu
