// C ABI of the MI355X HSTU jagged attention forward library: argument validation, variant
// selection and launch.  Host-side counterpart of the reference's adapter checks
// (ascendc/attention/hstu_v1/torch_extension/hstu_jagged_plugin.cpp:29-51,
//  ascendc/attention/hstu_v1/torch_extension/hstu_common.h:68-82) and of its host tiling
// (ascendc/attention/hstu_v1/hstu_forward_v1/op_host/tiling_policy_jagged.cpp:103-203,
//  ascendc/attention/hstu_v1/hstu_forward_v1/op_host/tiling_policy.cpp:68-93).
#include "../../include/hstu_mi355.h"

#include <hip/hip_runtime.h>
#include <stdlib.h>

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "hstu_clear.hip.h"
#include "hstu_error.h"
#include "hstu_variants.h"

namespace {
thread_local char g_err[512] = "";
}

// Scratch of the entry point that allocates nothing (hstu_jagged_fwd_noalloc): the workspace a caller of
// hstu_jagged_fwd would bring -- the counter block and one fp32 partial output per resident workgroup of the split
// variant (256 compute units: 512 x 64 KiB at head dim 128, 256 x 128 KiB at 256) -- as a device array of the
// library.  Every GPU the library runs on holds its own copy, at its own address, until the process ends.
constexpr uint64_t kScratchBytes = (32ull << 20) + hstu::kCounterBlockBytes;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

int hstu::set_error(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

namespace {

using hstu::BwdVariant;
using hstu::Variant;

#define fail(...) hstu::set_error(__VA_ARGS__)


// compute units of each device, looked up once
int compute_units(int* out)
{
    static int cached[64] = {0};
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) {
        return fail(HSTU_ERR_RUNTIME, "hipGetDevice failed: %s", hipGetErrorString(err));
    }
    if (dev < 0 || dev >= 64) {
        dev = 0;
    }
    if (cached[dev] == 0) {
        int n = 0;
        err = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
        if (err != hipSuccess || n <= 0) {
            return fail(HSTU_ERR_RUNTIME, "cannot read the number of compute units: %s", hipGetErrorString(err));
        }
        cached[dev] = n;
    }
    *out = cached[dev];
    return HSTU_OK;
}


// Process-wide switches.  They are read from the environment once, at the first call that looks at one, and again
// only when hstu_reload_switches() is called (a test that changes the environment calls it); a launch reads no
// environment variable.  A value of -1 means "not set: the library's own rule applies".
//   HSTU_MI355_SPLIT=0             forward: never cut long items into parts (the rows of a sequence are then the same bits
//                                  whatever else is in the batch)
//   HSTU_MI355_SHORT=0 / 1         forward: never / whenever possible the kernel for short lists
//   HSTU_MI355_GENERIC_BACKWARD=1  backward: the generic kernels also where tuned ones exist (for comparisons)
//   HSTU_MI355_BWD_HANDOFF=0/1/2   backward: force the launch order (two launches / three / planes)
//   HSTU_MI355_BWD_WORKSPACE_MB=n  backward: the largest workspace the library asks for
//   HSTU_MI355_BWD_PAIR_MAJOR=0/1  backward: the grids of the tuned 16-bit kernels level after level / pair after pair
struct Switches {
    int split;
    int short_lists;
    int generic_backward;
    int bwd_handoff;
    long long bwd_workspace_mb;
    int bwd_pair_major;
};
Switches g_switches = {-1, -1, -1, -1, -1, -1};
std::once_flag g_switches_once;

int switch_digit(const char* name, int max_digit)
{
    const char* const v = getenv(name);
    if (v == nullptr || v[0] < '0' || v[0] > '0' + max_digit || v[1] != '\0') {
        return -1;  // unset, empty or not one of the values the switch knows: the library's own rule
    }
    return v[0] - '0';
}
void read_switches()
{
    g_switches.split = switch_digit("HSTU_MI355_SPLIT", 1);
    g_switches.short_lists = switch_digit("HSTU_MI355_SHORT", 1);
    g_switches.generic_backward = switch_digit("HSTU_MI355_GENERIC_BACKWARD", 1);
    g_switches.bwd_handoff = switch_digit("HSTU_MI355_BWD_HANDOFF", 2);
    const char* const mb = getenv("HSTU_MI355_BWD_WORKSPACE_MB");
    g_switches.bwd_workspace_mb = (mb != nullptr && mb[0] >= '0' && mb[0] <= '9') ? atoll(mb) : -1;
    g_switches.bwd_pair_major = switch_digit("HSTU_MI355_BWD_PAIR_MAJOR", 1);
}
const Switches& switches()
{
    std::call_once(g_switches_once, read_switches);
    return g_switches;
}
// The largest backward workspace the library asks for, in MiB.  HSTU_MI355_BWD_WORKSPACE_MB sets it for every call.
// Otherwise 2 GiB -- a training step has better uses for its memory than the last few per cent of this operator, and a
// call whose planes would need more runs on the two-launch order, which needs none -- except where more buys a good part
// of the call (`large`: 16-bit inputs at head dims above 128, where a product is dearest; plan_bwd takes more than the
// 2 GiB only for an estimated tenth of the time): 16 GiB of an MI355X's 288 GB.  With 2 GiB everywhere, 32 x 8 heads of
// 4096 rows at d 256 took 15.5 ms, 11.0 ms with their 8.7 GB of planes; 64 x 4 heads of 1024..4096 rows 7.9 -> 4.7 ms.
int64_t workspace_cap_mb(bool large = false)
{
    const long long set = switches().bwd_workspace_mb;
    return set >= 0 ? static_cast<int64_t>(set) : (large ? 16384 : 2048);
}


int validate(const hstu_jagged_fwd_params* p, bool need_out = true)
{
    if (p == nullptr) {
        return fail(HSTU_ERR_NULLPTR, "params is NULL");
    }
    if (p->struct_size != sizeof(hstu_jagged_fwd_params)) {
        return fail(HSTU_ERR_INVALID, "struct_size %u does not match this library (%zu)", p->struct_size,
                    sizeof(hstu_jagged_fwd_params));
    }
    if (p->n_offsets < 2) {
        return fail(HSTU_ERR_INVALID, "seq_offset params error should have at least two element.");
    }
    const int64_t batch = p->n_offsets - 1;
    if (batch > HSTU_MAX_BATCH) {
        return fail(HSTU_ERR_INVALID, "batchSize limit (0, %d], but get %lld", HSTU_MAX_BATCH, (long long)batch);
    }
    if (p->max_seq_len_q < 1 || p->max_seq_len_q > HSTU_MAX_SEQ_LEN) {
        return fail(HSTU_ERR_INVALID, "maxSeqLen expect in [1, 20480], but value is %lld",
                    (long long)p->max_seq_len_q);
    }
    if (p->max_seq_len_k < 1 || p->max_seq_len_k > HSTU_MAX_SEQ_LEN) {
        return fail(HSTU_ERR_INVALID, "maxSeqLenK expect in [1, 20480], but value is %lld",
                    (long long)p->max_seq_len_k);
    }
    if (p->mask_type < HSTU_MASK_TRIL || p->mask_type > HSTU_MASK_CUSTOM) {
        return fail(HSTU_ERR_INVALID, "maskType expect in [0, 3], but value is %lld", (long long)p->mask_type);
    }
    if (p->mask_type == HSTU_MASK_TRIU) {
        return fail(HSTU_ERR_INVALID, "maskType current not support triu now, pls use custome mask");
    }
    if (p->mask_type == HSTU_MASK_CUSTOM && p->mask == nullptr) {
        return fail(HSTU_ERR_INVALID, "use custome mask must have valide mask tensor");
    }
    if (p->total_q < 0 || p->total_k < 0) {
        return fail(HSTU_ERR_INVALID, "negative row count");
    }
    if (p->num_heads_q < 1 || p->num_heads_q > HSTU_MAX_HEADS || p->num_heads_k < 1 ||
        p->num_heads_k > HSTU_MAX_HEADS) {
        return fail(HSTU_ERR_INVALID, "head num expect in [1, %d], but q has %lld and k has %lld", HSTU_MAX_HEADS,
                    (long long)p->num_heads_q, (long long)p->num_heads_k);
    }
    if (p->num_heads_q % p->num_heads_k != 0) {
        return fail(HSTU_ERR_INVALID, "For GQA, headNumQ must be divisible by headNumK");
    }
    if (p->head_dim_qk < 1 || p->head_dim_qk > HSTU_MAX_HEAD_DIM) {
        return fail(HSTU_ERR_INVALID, "dim size expect in [1, 512], but q/k head dim is %lld",
                    (long long)p->head_dim_qk);
    }
    if (p->head_dim_v < 16 || p->head_dim_v > HSTU_MAX_HEAD_DIM || p->head_dim_v % 16 != 0) {
        return fail(HSTU_ERR_INVALID, "dim size expect in [16, 512] step 16, but v head dim is %lld",
                    (long long)p->head_dim_v);
    }
    if (p->target_group_size < 0) {
        return fail(HSTU_ERR_INVALID, "targetGroupSize must be >= 0");
    }
    if (p->index_dtype != HSTU_IDX_I32 && p->index_dtype != HSTU_IDX_I64) {
        return fail(HSTU_ERR_INVALID, "index_dtype must be int32 or int64");
    }
    if (p->dtype < HSTU_DT_BF16 || p->dtype > HSTU_DT_FP8_E4M3) {
        return fail(HSTU_ERR_INVALID, "unknown dtype %d", p->dtype);
    }
    const bool empty = (p->total_q == 0);
    if (!empty && (p->q == nullptr || (need_out && p->out == nullptr))) {
        return fail(HSTU_ERR_NULLPTR, "q / out must not be NULL");
    }
    if (p->total_k > 0 && (p->k == nullptr || p->v == nullptr)) {
        return fail(HSTU_ERR_NULLPTR, "k / v must not be NULL");
    }
    if (p->seq_offset_q == nullptr || p->seq_offset_k == nullptr) {
        return fail(HSTU_ERR_NULLPTR, "seq_offset_q / seq_offset_k must not be NULL");
    }
    return HSTU_OK;
}

// picks the kernel variant; returns nullptr (and sets the error) when the combination is not built
const Variant* select(const hstu_jagged_fwd_params* p)
{
    if (p->dtype == HSTU_DT_FP8_E4M3) {
        if (p->out_dtype != HSTU_DT_FP16 && p->out_dtype != HSTU_DT_BF16) {
            fail(HSTU_ERR_UNSUPPORTED, "fp8 inputs produce fp16 (the reference's choice) or bf16 output");
            return nullptr;
        }
    } else if (p->out_dtype != p->dtype) {
        fail(HSTU_ERR_UNSUPPORTED, "out_dtype must equal dtype for bf16 / fp16 / fp32 inputs");
        return nullptr;
    }
    const int64_t dmax = p->head_dim_qk > p->head_dim_v ? p->head_dim_qk : p->head_dim_v;
    // The tuned kernels take head dims up to 256 with a q/k head dim that is a multiple of 8 (16-byte chunks), and
    // address one sequence of one head group through a 32-bit buffer descriptor, with room above it for the offsets
    // that mark a request as out of range.  Whatever else the reference accepts (head dims up to 512, any q/k head
    // dim) goes to the kernel written for coverage.
    const int64_t esize = p->dtype == HSTU_DT_FP32 ? 4 : (p->dtype == HSTU_DT_FP8_E4M3 ? 1 : 2);
    const int64_t span_q = p->max_seq_len_q * p->num_heads_q * dmax * esize;
    const int64_t span_k = p->max_seq_len_k * p->num_heads_k * dmax * esize;
    const int64_t span_b = p->max_seq_len_q * p->max_seq_len_k * esize;
    const bool wide_span = span_q >= (1LL << 30) || span_k >= (1LL << 30) ||
                           ((p->attn_bias != nullptr || p->mask_type == HSTU_MASK_CUSTOM) && span_b >= (1LL << 31));
    if ((p->dtype == HSTU_DT_BF16 || p->dtype == HSTU_DT_FP16) && dmax > 256 && p->head_dim_qk % 8 == 0) {
        // head dims in (256, 512]: the matrix-pipe kernel without the tuned kernel's pipeline (one sequence of one head
        // group behind a 32-bit descriptor at the padded head dim 512)
        const int64_t wide_q = p->max_seq_len_q * p->num_heads_q * 512 * 2;
        const int64_t wide_k = p->max_seq_len_k * p->num_heads_k * 512 * 2;
        if (wide_q < (1LL << 30) && wide_k < (1LL << 30) && !wide_span) {
            return &hstu::fwd_variants_wide()[p->dtype == HSTU_DT_BF16 ? 0 : 1][p->attn_bias != nullptr ? 1 : 0]
                                             [p->mask_type == HSTU_MASK_CUSTOM ? 1 : 0];
        }
    }
    // (the tuned fp8 kernels read 16-byte chunks of one-byte elements: a q/k head dim that is a multiple of 16)
    const bool odd_f8 = p->dtype == HSTU_DT_FP8_E4M3 && p->head_dim_qk % 16 != 0;
    if (p->head_dim_qk % 8 != 0 || dmax > 256 || wide_span || odd_f8) {
        if (p->dtype == HSTU_DT_FP8_E4M3) {
            return &hstu::fwd_variants_generic()[p->out_dtype == HSTU_DT_FP16 ? 3 : 4];
        }
        return &hstu::fwd_variants_generic()[p->dtype == HSTU_DT_BF16 ? 0 : (p->dtype == HSTU_DT_FP16 ? 1 : 2)];
    }
    const int slot = dmax <= 32 ? 0 : (dmax <= 64 ? 1 : (dmax <= 128 ? 2 : 3));
    if (p->dtype == HSTU_DT_FP8_E4M3) {
        return &hstu::fwd_variants_f8()[p->out_dtype == HSTU_DT_FP16 ? 0 : 1][p->attn_bias != nullptr ? 1 : 0]
                                        [p->mask_type == HSTU_MASK_CUSTOM ? 1 : 0][slot <= 1 ? 0 : slot - 1];
    }
    if (p->dtype == HSTU_DT_FP32) {
        return &hstu::fwd_variants_f32()[p->attn_bias != nullptr ? 1 : 0][p->mask_type == HSTU_MASK_CUSTOM ? 1 : 0][slot];
    }
    const auto* table = p->dtype == HSTU_DT_BF16 ? hstu::fwd_variants_bf16() : hstu::fwd_variants_f16();
    return &table[p->attn_bias != nullptr ? 1 : 0][p->mask_type == HSTU_MASK_CUSTOM ? 1 : 0][slot];
}

// The kernel for batches of tiny sequences (hstu_fwd_tiny_kernel.hip.h): 16-bit inputs with head dims up to 256 (q/k head
// dim a multiple of 8) without bias or custom mask, no sequence longer than 64 rows or keys, 16-byte aligned tensors.
// Batch 2048 x 2 heads x 32 rows at head dim 256: 135 us on the persistent kernel (a 128-row workgroup and its start-up
// per item); batch 2048 x 4 heads x 48 rows at head dim 64: 118 us.  HSTU_MI355_SHORT=0 switches it off with the kernel
// for short lists.
const hstu::ShortVariant* tiny_variant(const Variant* var, const hstu_jagged_fwd_params* p, unsigned* threads)
{
    const int64_t dmax = p->head_dim_qk > p->head_dim_v ? p->head_dim_qk : p->head_dim_v;
    const uintptr_t ptrs = reinterpret_cast<uintptr_t>(p->q) | reinterpret_cast<uintptr_t>(p->k) | reinterpret_cast<uintptr_t>(p->v);
    if ((p->dtype != HSTU_DT_BF16 && p->dtype != HSTU_DT_FP16) || p->attn_bias != nullptr || p->mask_type == HSTU_MASK_CUSTOM ||
        dmax > 256 || p->head_dim_qk % 8 != 0 || p->head_dim_v % 8 != 0 || ptrs % 16 != 0 || var->persistent_wgs_per_cu <= 0 ||
        p->max_seq_len_q > 64 || p->max_seq_len_k > 64 || switches().short_lists == 0) {
        return nullptr;
    }
    const int rows64 = (p->max_seq_len_q > 32 || p->max_seq_len_k > 32) ? 1 : 0;
    *threads = rows64 ? 256u : 128u;
    return &hstu::fwd_variants_tiny()[p->dtype == HSTU_DT_BF16 ? 0 : 1][dmax <= 64 ? 0 : (dmax <= 128 ? 1 : 2)][rows64];
}

// The kernel for small launches of sequences with few query rows (hstu_fwd_few_rows_kernel.hip.h): 16-bit inputs with head
// dims up to 128 (q/k head dim a multiple of 8), no bias, no custom mask, no sequence of more than 64 query rows (keys:
// any number), 16-byte aligned tensors, and at most one (sequence, head) item per compute unit -- a launch then lasts
// as long as one item, whose keys the kernel deals over the wavefronts of a workgroup; with more items the persistent
// kernel, which streams K and V at the rate of memory, is the faster one.  HSTU_MI355_SHORT=0 switches it off.
const hstu::ShortVariant* few_rows_variant(const Variant* var, const hstu_jagged_fwd_params* p)
{
    const int64_t dmax = p->head_dim_qk > p->head_dim_v ? p->head_dim_qk : p->head_dim_v;
    const uintptr_t ptrs = reinterpret_cast<uintptr_t>(p->q) | reinterpret_cast<uintptr_t>(p->k) | reinterpret_cast<uintptr_t>(p->v);
    const int64_t span_k = p->max_seq_len_k * p->num_heads_k * dmax * 2;
    if ((p->dtype != HSTU_DT_BF16 && p->dtype != HSTU_DT_FP16) || p->attn_bias != nullptr || p->mask_type == HSTU_MASK_CUSTOM ||
        dmax > 128 || p->head_dim_qk % 8 != 0 || p->head_dim_v % 8 != 0 || ptrs % 16 != 0 || var->persistent_wgs_per_cu <= 0 ||
        p->max_seq_len_q > hstu::kFewRows || span_k >= (1LL << 30) || switches().short_lists == 0) {
        return nullptr;
    }
    int cus = 0;
    if (compute_units(&cus) != HSTU_OK || (p->n_offsets - 1) * p->num_heads_q > cus) {
        return nullptr;
    }
    // ... and few sub-tiles per wavefront: the row groups of an item each fetch the item's K and V, which the persistent
    // kernel shares through LDS (and long items it splits over workgroups).  Measured, fp16, this kernel against that one:
    // 16 x 4 heads, 32 rows x 499 keys, d 64 / 32: 10.7 / 14.4 us; 16 rows x 1000 keys: 10.9 / 20.0; 32 x 8 heads, 10 x 500:
    // 8.7 / 14.4; 256 x 1 head, 52 x 1000: 24.0 / 29.5; 8 x 8 heads, d 128, 32 x 2000 (16 sub-tiles per wavefront): 40.6 /
    // 37.9; 64 x 4 heads, d 64, 64 x 4096 (64 per wavefront): 87.2 / 61.7
    const int64_t splits = p->max_seq_len_q <= 16 ? 8 : (p->max_seq_len_q <= 32 ? 4 : 2);
    const int64_t per_wavefront = ((p->max_seq_len_k + 31) / 32 + splits - 1) / splits;
    if (per_wavefront > (dmax <= 64 ? 16 : 8)) {
        return nullptr;
    }
    return &hstu::fwd_variants_few_rows()[p->dtype == HSTU_DT_BF16 ? 0 : 1][dmax <= 64 ? 0 : 1];
}
// the kernels with one workgroup per (sequence, head) item: tiny sequences first, then few query rows
const hstu::ShortVariant* one_item_variant(const Variant* var, const hstu_jagged_fwd_params* p, unsigned* threads)
{
    if (const hstu::ShortVariant* const tv = tiny_variant(var, p, threads)) {
        return tv;
    }
    *threads = hstu::kFwdFewRowsThreads;
    return few_rows_variant(var, p);
}

// The kernel for short work lists (hstu_fwd_short_kernel.hip.h) takes 16-bit inputs at the head-dim slot 128 without
// bias or custom mask.  It is the faster one while the list -- at most n_blocks entries -- is a few items per
// workgroup the persistent kernel would keep resident: there a launch lasts as long as its longest item, which the
// short kernel's narrower wavefronts finish in about half the time; on longer lists the persistent kernel's
// steady-state rate wins.  HSTU_MI355_SHORT in the environment overrides the rule: 0 = never, 1 = whenever the
// kernel can take the call.
const hstu::ShortVariant* short_variant(const Variant* var, const hstu_jagged_fwd_params* p, bool have_counters = true)
{
    if ((p->dtype != HSTU_DT_BF16 && p->dtype != HSTU_DT_FP16) || p->mask_type == HSTU_MASK_CUSTOM || var->d_pad != 128 ||
        var->persistent_wgs_per_cu <= 0 || var->kernel_queues == nullptr) {
        return nullptr;
    }
    unsigned one_item_threads = 0;
    if (one_item_variant(var, p, &one_item_threads) != nullptr) {
        return nullptr;
    }
    // (with a bias: rows of 8-byte pieces)
    const bool bias = p->attn_bias != nullptr;
    if (bias && (p->max_seq_len_k % 4 != 0 || reinterpret_cast<uintptr_t>(p->attn_bias) % 8 != 0 ||
                 p->max_seq_len_q * p->max_seq_len_k * 2 >= (1LL << 32))) {
        return nullptr;
    }
    const hstu::ShortVariant* const sv = &hstu::fwd_variants_short()[(bias ? 2 : 0) + (p->dtype == HSTU_DT_BF16 ? 0 : 1)];
    const int forced = switches().short_lists;
    if (forced == 0) {
        return nullptr;
    }
    if (forced == 1) {
        return sv;
    }
    int cus = 0;
    if (compute_units(&cus) != HSTU_OK) {
        return nullptr;
    }
    // Measured on MI355X (bf16, head dim 128, persistent kernel -> this one): keys up to 1024 -- batch 32 x 4 heads
    // lengths 256..1024 37.4 -> 35.0 us, 8 x 4 of 1024 32.9 -> 25.2, 64 x 4 of 512 43.1 -> 39.3, 256 x 4 of 256
    // 68.2 -> 53.2, 2048 x 2 of 32 71.0 -> 40.0, 128 x 4 of 1024 220.9 -> 217.3 (even); keys up to 2048 with one to
    // two slots per resident workgroup -- 8 x 8 of 1536 62.5 -> 52.5, 8 x 4 of 2048 57.4 -> 51.5, 16 x 4 of 2048 even;
    // beyond that the persistent kernel's variants win: 32 x 4 lengths 512..2048 103.7 -> 107.9, 4 x 2 of 2048 36.7
    // (split items) -> 41.4, 16 x 4 of 4096 291 -> 296, 1 x 4 of 8192 127 (split) -> 177.
    const int64_t resident = static_cast<int64_t>(cus) * var->persistent_wgs_per_cu;
    const int64_t n_qtiles = (p->max_seq_len_q + hstu::kBlockM - 1) / hstu::kBlockM;
    const int64_t n_blocks = n_qtiles * (p->n_offsets - 1) * p->num_heads_q;
    if (bias) {
        // with an attn_bias: keys up to 1024 and at most one slot per resident workgroup -- 8 x 4 of 1024 36.6 -> 27.6 us,
        // 16 x 4 lengths 512..1024 45.0 -> 38.4; two slots per workgroup are even (32 x 4 lengths 256..1024, 64 x 4 of 512)
        // and longer rows lose (16 x 4 lengths 512..2048 64 -> 84 us, 8 x 8 lengths 1024..2048 80 -> 98)
        return (p->max_seq_len_k <= 1024 && n_blocks <= resident) ? sv : nullptr;
    }
    // Long lists over more K / V rows than the caches hold go to the persistent kernel's queues, which take the items pair
    // after pair on one XCD each: this kernel's grid runs level after level, so that every resident workgroup then streams
    // another pair's keys from memory.  (This kernel -> the queues, 4 heads, lengths 256..1024: batch 128 112 -> 117 us, 256
    // 237 -> 232, 384 431 -> 370, 512 629 -> 449; 256 x 1024 rows 557 -> 398, 512 x 512 rows 371 -> 288, 1024 x 64..512 rows
    // 408 -> 335; sequences of a tile or two have nothing to share: 2048 x 16..256 rows 282 -> 299.)
    const int64_t batch = p->n_offsets - 1;
    const int64_t items = (p->total_q / hstu::kBlockM + batch / 2) * p->num_heads_q;  // (by the mean length)
    const int64_t kv_bytes = p->total_k * p->num_heads_k * (p->head_dim_qk + p->head_dim_v) * 2;
    // (a caller that brings no room for the queues' counters keeps this kernel: the plain list runs level after level too)
    if (have_counters && items >= 6 * resident && kv_bytes >= (256LL << 20) && p->total_q >= 256 * batch) {
        return nullptr;
    }
    const bool short_keys = p->max_seq_len_k <= 1024;
    const bool one_round = p->max_seq_len_k <= 2048 && n_blocks >= resident && n_blocks <= 2 * resident;
    return (short_keys || one_round) ? sv : nullptr;
}

// persistent workgroups per CU of a launch: what the variant is compiled for, except that the slot-32 variants with a
// bias or a custom mask, compiled for three, are launched two per CU when rows are longer than 2048 keys -- there the
// bias stream is the bound and a third reader per CU costs 3 % (B32 H8 L4096 1351 -> 1391 us), where it is worth
// 9 % at L1024 (98.5 -> 89.2 us) and 1 % at L2048
int wgs_per_cu(const Variant* var, const hstu_jagged_fwd_params* p)
{
    const bool biased = p->attn_bias != nullptr || p->mask_type == HSTU_MASK_CUSTOM;
    if (biased && var->d_pad <= 32 && var->persistent_wgs_per_cu == 3 && p->max_seq_len_k > 2048) {
        return 2;
    }
    return var->persistent_wgs_per_cu;
}

// whether the launch described by p takes the variant with per-XCD work queues: only when the list may hold
// several items per resident workgroup.  *resident_out (optional) receives the resident grid.
bool takes_queue_variant(const Variant* var, const hstu_jagged_fwd_params* p, int64_t* resident_out)
{
    if (var->persistent_wgs_per_cu <= 0) {
        return false;
    }
    int cus = 0;
    if (compute_units(&cus) != HSTU_OK) {
        return false;
    }
    const int64_t resident = static_cast<int64_t>(cus) * wgs_per_cu(var, p);
    if (resident_out != nullptr) {
        *resident_out = resident;
    }
    const int64_t n_qtiles = (p->max_seq_len_q + hstu::kBlockM - 1) / hstu::kBlockM;
    const int64_t n_blocks = n_qtiles * (p->n_offsets - 1) * p->num_heads_q;
    return var->kernel_queues != nullptr && n_blocks >= 4 * resident;
}

// Split items: a list that cannot have two items per resident workgroup takes the variant that may cut long items
// into parts (it does so when there are fewer items than workgroups), if the caller brings a workspace.  Behind the
// counter block the workspace holds the fp32 partial outputs, kBlockM x d_pad floats each; room for one per resident
// workgroup is asked for: the kernel never lists more entries than there are workgroups when it splits, and splits
// only as far as the room goes.
constexpr uint64_t kMaxWorkspaceBytes = 128ull << 20;
constexpr uint64_t kCounterBytes = hstu::kCounterBlockBytes;  // head of the workspace of the variants that pull from counters
uint64_t split_part_bytes(const Variant* var) { return static_cast<uint64_t>(hstu::kBlockM) * var->d_pad * sizeof(float); }
bool may_take_split_variant(const Variant* var, const hstu_jagged_fwd_params* p, int64_t* resident_out)
{
    if (var->persistent_wgs_per_cu <= 0 || var->kernel_split == nullptr) {
        return false;
    }
    // HSTU_MI355_SPLIT=0 turns splitting off: the rows of a sequence then come out bit for bit the same whatever
    // else is in the batch (a split changes the order of the fp32 sums)
    if (switches().split == 0) {
        return false;
    }
    int cus = 0;
    if (compute_units(&cus) != HSTU_OK) {
        return false;
    }
    const int64_t resident = static_cast<int64_t>(cus) * wgs_per_cu(var, p);
    if (resident_out != nullptr) {
        *resident_out = resident;
    }
    const int64_t n_qtiles = (p->max_seq_len_q + hstu::kBlockM - 1) / hstu::kBlockM;
    const int64_t n_blocks = n_qtiles * (p->n_offsets - 1) * p->num_heads_q;
    // (items of at most 16 sub-tiles: parts of 8, the kernel's shortest, do not earn back what a part costs --
    // 8 x 4 sequences of 512 rows: 23.0 us split, 20.7 us not)
    return n_blocks < 2 * resident && p->max_seq_len_k > 16 * 32;
}
uint64_t split_workspace_bytes(const Variant* var, const hstu_jagged_fwd_params* p)
{
    int64_t resident = 0;
    if (!may_take_split_variant(var, p, &resident)) {
        return 0;
    }
    const uint64_t bytes = kCounterBytes + static_cast<uint64_t>(resident) * split_part_bytes(var);
    return bytes < kMaxWorkspaceBytes ? bytes : kMaxWorkspaceBytes;
}

// what a forward launch described by p asks of its caller: the counter block when the list may be long enough for
// the variant with per-XCD queues, the counter block and room for partial outputs when it may be short enough to
// split items, nothing for the lists in between (fixed schedule, no device counters)
uint64_t forward_workspace_bytes(const Variant* var, const hstu_jagged_fwd_params* p)
{
    unsigned one_item_threads = 0;
    if (short_variant(var, p) != nullptr || one_item_variant(var, p, &one_item_threads) != nullptr) {
        return 0;
    }
    if (takes_queue_variant(var, p, nullptr)) {
        return kCounterBytes;
    }
    return split_workspace_bytes(var, p);
}

bool usable_workspace(const void* workspace, uint64_t bytes, uint64_t need)
{
    return workspace != nullptr && bytes >= need && reinterpret_cast<uintptr_t>(workspace) % 16 == 0;
}

// ---- backward -------------------------------------------------------------------------------------------

// clears the attn_bias gradient when the key-tile kernel, which does it beside its work, is not launched
__global__ __launch_bounds__(256) void hstu_clear_kernel(void* p, int64_t n_bytes)
{
    hstu::clear_share(p, n_bytes, blockIdx.x, gridDim.x, static_cast<int>(threadIdx.x), 256);
}
void launch_clear(void* p, int64_t n_bytes, void* stream)
{
    const int64_t want = (n_bytes + 256 * 16 * 8 - 1) / (256 * 16 * 8);  // eight pieces per thread
    const unsigned grid = static_cast<unsigned>(want < 1 ? 1 : (want > 4096 ? 4096 : want));
    hipLaunchKernelGGL(hstu_clear_kernel, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream), p, n_bytes);
}

int validate_bwd(const hstu_jagged_bwd_params* p)
{
    if (p == nullptr) {
        return fail(HSTU_ERR_NULLPTR, "params is NULL");
    }
    if (p->struct_size != sizeof(hstu_jagged_bwd_params)) {
        return fail(HSTU_ERR_INVALID, "struct_size %u does not match this library (%zu)", p->struct_size,
                    sizeof(hstu_jagged_bwd_params));
    }
    const int rc = validate(&p->fwd, false);
    if (rc != HSTU_OK) {
        return rc;
    }
    if (p->fwd.total_q > 0 && (p->grad == nullptr || p->grad_q == nullptr)) {
        return fail(HSTU_ERR_NULLPTR, "grad / grad_q must not be NULL");
    }
    if (p->fwd.total_k > 0 && (p->grad_k == nullptr || p->grad_v == nullptr)) {
        return fail(HSTU_ERR_NULLPTR, "grad_k / grad_v must not be NULL");
    }
    if (p->grad_attn_bias != nullptr && p->fwd.attn_bias == nullptr) {
        return fail(HSTU_ERR_INVALID, "grad_attn_bias without attn_bias");
    }
    return HSTU_OK;
}

// the generic and the fp32 variants: one workgroup per key tile, outputs cleared by fills ahead of the two kernels
bool is_generic_bwd(const BwdVariant* v)
{
    const BwdVariant* g = &hstu::bwd_variants_generic()[0][0];
    const BwdVariant* f = &hstu::bwd_variants_f32()[0][0][0];
    return (v >= g && v < g + 9) || (v >= f && v < f + 12);
}

// The tuned kernels take bf16 / fp16 with head dims up to 256, a q/k head dim that is a multiple of 8 and sequences
// whose rows span less than 1 GiB (32-bit offsets); everything else the reference's backward accepts (fp32, head
// dims up to 512, any q/k head dim) runs on the generic kernels, which HSTU_MI355_GENERIC_BACKWARD=1 in the
// environment also selects for inputs the tuned kernels would take (for comparisons).
const BwdVariant* select_bwd(const hstu_jagged_bwd_params* p)
{
    const hstu_jagged_fwd_params* f = &p->fwd;
    if (f->dtype != HSTU_DT_BF16 && f->dtype != HSTU_DT_FP16 && f->dtype != HSTU_DT_FP32) {
        fail(HSTU_ERR_UNSUPPORTED, "the backward is built for bf16, fp16 and fp32");
        return nullptr;
    }
    const int64_t dmax = f->head_dim_qk > f->head_dim_v ? f->head_dim_qk : f->head_dim_v;
    const BwdVariant* generic = &hstu::bwd_variants_generic()[f->dtype == HSTU_DT_BF16 ? 0 : (f->dtype == HSTU_DT_FP16 ? 1 : 2)]
                                                             [dmax <= 128 ? 0 : (dmax <= 256 ? 1 : 2)];
    const bool force_generic = switches().generic_backward == 1;
    if (f->dtype == HSTU_DT_FP32 && dmax <= 128 && f->head_dim_qk % 8 == 0 && !force_generic) {
        // fp32 MFMA kernels: one sequence of one head group behind a 32-bit descriptor
        const int64_t sq4 = f->max_seq_len_q * f->num_heads_q * dmax * 4;
        const int64_t sk4 = f->max_seq_len_k * f->num_heads_k * dmax * 4;
        const int64_t sb4 = f->max_seq_len_q * f->max_seq_len_k * 4;
        if (sq4 < (1LL << 30) && sk4 < (1LL << 30) &&
            !((f->attn_bias != nullptr || f->mask_type == HSTU_MASK_CUSTOM) && sb4 >= (1LL << 31))) {
            return &hstu::bwd_variants_f32()[f->attn_bias != nullptr ? 1 : 0][f->mask_type == HSTU_MASK_CUSTOM ? 1 : 0]
                                            [dmax <= 32 ? 0 : (dmax <= 64 ? 1 : 2)];
        }
    }
    if (f->dtype == HSTU_DT_FP32 || dmax > 256 || f->head_dim_qk % 8 != 0) {
        return generic;
    }
    const int64_t span_q = f->max_seq_len_q * f->num_heads_q * dmax * 2;
    const int64_t span_k = f->max_seq_len_k * f->num_heads_k * dmax * 2;
    const int64_t span_b = f->max_seq_len_q * f->max_seq_len_k * 2;
    if (span_q >= (1LL << 30) || span_k >= (1LL << 30) ||
        ((f->attn_bias != nullptr || f->mask_type == HSTU_MASK_CUSTOM) && span_b >= (1LL << 31))) {
        return generic;
    }
    if (force_generic) {
        return generic;
    }
    const auto* table = f->dtype == HSTU_DT_BF16 ? hstu::bwd_variants_bf16() : hstu::bwd_variants_f16();
    return &table[f->attn_bias != nullptr ? 1 : 0][f->mask_type == HSTU_MASK_CUSTOM ? 1 : 0][dmax <= 64 ? 0 : (dmax <= 128 ? 1 : 2)];
}

// ---- paged K/V --------------------------------------------------------------------------------------------
int launch_forward(const hstu_jagged_fwd_params* p, const hstu_paged_fwd_params* paged, void* workspace,
                   uint64_t workspace_bytes, void* stream);

uint64_t round_up_256(uint64_t x) { return (x + 255u) & ~static_cast<uint64_t>(255u); }

int validate_paged(const hstu_paged_fwd_params* p, hstu_jagged_fwd_params* gathered, uint64_t* region_bytes)
{
    if (p == nullptr) {
        return fail(HSTU_ERR_NULLPTR, "params is NULL");
    }
    if (p->struct_size != sizeof(hstu_paged_fwd_params)) {
        return fail(HSTU_ERR_INVALID, "struct_size %u does not match this library (%zu)", p->struct_size,
                    sizeof(hstu_paged_fwd_params));
    }
    const int rc = validate(&p->fwd);
    if (rc != HSTU_OK) {
        return rc;
    }
    if (p->kv_cache == nullptr || p->page_offsets == nullptr || p->page_ids == nullptr) {
        return fail(HSTU_ERR_NULLPTR, "kv_cache / page_offsets / page_ids must not be NULL");
    }
    if (p->page_size != 32 && p->page_size != 64 && p->page_size != 128 && p->page_size != 256) {
        return fail(HSTU_ERR_INVALID, "page_size must be 32, 64, 128 or 256, but value is %lld", (long long)p->page_size);
    }
    if (p->num_pages < 1 || p->n_page_ids < 1) {
        return fail(HSTU_ERR_INVALID, "kv_cache and page_ids must not be empty");
    }
    if (p->fwd.dtype == HSTU_DT_FP8_E4M3) {
        fail(HSTU_ERR_UNSUPPORTED, "paged K/V is not built for fp8 inputs");
        return HSTU_ERR_UNSUPPORTED;
    }
    if (p->fwd.head_dim_qk != p->fwd.head_dim_v) {
        return fail(HSTU_ERR_INVALID, "the cache holds K and V rows of one head dim, but q/k has %lld and v has %lld",
                    (long long)p->fwd.head_dim_qk, (long long)p->fwd.head_dim_v);
    }
    const uint64_t esize = p->fwd.dtype == HSTU_DT_FP32 ? 4 : 2;
    const uint64_t row_bytes = static_cast<uint64_t>(p->fwd.num_heads_k) * p->fwd.head_dim_qk * esize;
    if (row_bytes % 16 != 0) {
        fail(HSTU_ERR_UNSUPPORTED, "a K/V row of %llu bytes is not a multiple of 16", (unsigned long long)row_bytes);
        return HSTU_ERR_UNSUPPORTED;
    }
    *region_bytes = round_up_256(static_cast<uint64_t>(p->fwd.total_k) * row_bytes);
    *gathered = p->fwd;
    gathered->num_context = nullptr;
    return HSTU_OK;
}

}  // namespace

extern "C" {

HSTU_API int hstu_paged_fwd_workspace_size(const hstu_paged_fwd_params* params, uint64_t* workspace_bytes)
{
    if (workspace_bytes == nullptr) {
        return fail(HSTU_ERR_NULLPTR, "workspace_bytes is NULL");
    }
    *workspace_bytes = 0;
    hstu_jagged_fwd_params g;
    uint64_t region = 0;
    const int rc = validate_paged(params, &g, &region);
    if (rc != HSTU_OK) {
        return rc;
    }
    const Variant* var = select(&g);
    if (var == nullptr) {
        return HSTU_ERR_UNSUPPORTED;
    }
    if (var->kernel_paged != nullptr) {
        // the kernel reads the pages itself; the counter block (required: the variant pulls its items from a
        // counter) and, for short lists, room for the partial outputs of split items (optional)
        const uint64_t split = split_workspace_bytes(var, &g);
        *workspace_bytes = split > kCounterBytes ? split : kCounterBytes;
        return HSTU_OK;
    }
    uint64_t inner = 0;
    const int rc2 = hstu_jagged_fwd_workspace_size(&g, &inner);
    if (rc2 != HSTU_OK) {
        return rc2;
    }
    *workspace_bytes = 2 * region + inner;
    return HSTU_OK;
}

HSTU_API int hstu_paged_fwd(const hstu_paged_fwd_params* p, void* workspace, uint64_t workspace_bytes, void* stream)
{
    hstu_jagged_fwd_params g;
    uint64_t region = 0;
    const int rc = validate_paged(p, &g, &region);
    if (rc != HSTU_OK) {
        return rc;
    }
    if (p->fwd.total_q == 0) {
        return HSTU_OK;
    }
    const Variant* var = select(&g);
    if (var == nullptr) {
        return HSTU_ERR_UNSUPPORTED;
    }
    if (var->kernel_paged != nullptr) {
        if (!usable_workspace(workspace, workspace_bytes, kCounterBytes)) {
            return fail(HSTU_ERR_WORKSPACE, "the paged forward needs a 16-byte aligned workspace of at least %llu bytes",
                        (unsigned long long)kCounterBytes);
        }
        return launch_forward(&g, p, workspace, workspace_bytes, stream);
    }
    // no paged kernel for this combination (fp32, head dims up to 32 or above 256): gather the rows, then the plain forward
    if (p->fwd.total_k > 0) {
        if (workspace == nullptr || workspace_bytes < 2 * region || reinterpret_cast<uintptr_t>(workspace) % 16 != 0) {
            return fail(HSTU_ERR_WORKSPACE, "the paged forward needs a 16-byte aligned workspace of at least %llu bytes",
                        (unsigned long long)(2 * region));
        }
        if (p->fwd.total_k > 0x7fffffffLL) {
            return fail(HSTU_ERR_INVALID, "too many key rows");
        }
        hstu::PagedGatherArgs a;
        memset(&a, 0, sizeof(a));
        a.k = p->fwd.k;
        a.v = p->fwd.v;
        a.kv_cache = p->kv_cache;
        a.k_out = workspace;
        a.v_out = static_cast<char*>(workspace) + region;
        a.offs_q = p->fwd.seq_offset_q;
        a.offs_k = p->fwd.seq_offset_k;
        a.page_offsets = p->page_offsets;
        a.page_ids = p->page_ids;
        a.num_tgt = p->fwd.num_target;
        a.total_q = p->fwd.total_q;
        a.total_k = p->fwd.total_k;
        a.num_pages = p->num_pages;
        a.n_page_ids = p->n_page_ids;
        a.n_batch = static_cast<int>(p->fwd.n_offsets - 1);
        a.page_size = static_cast<int>(p->page_size);
        a.row_bytes = static_cast<int>(p->fwd.num_heads_k * p->fwd.head_dim_qk * (p->fwd.dtype == HSTU_DT_FP32 ? 4 : 2));
        a.idx64 = (p->fwd.index_dtype == HSTU_IDX_I64) ? 1 : 0;
        hstu::launch_paged_gather(a, static_cast<unsigned>(p->fwd.total_k), static_cast<hipStream_t>(stream));
        const hipError_t err = hipGetLastError();
        if (err != hipSuccess) {
            return fail(HSTU_ERR_RUNTIME, "launch of the paged gather failed: %s", hipGetErrorString(err));
        }
        g.k = workspace;
        g.v = static_cast<char*>(workspace) + region;
    }
    const uint64_t used = p->fwd.total_k > 0 ? 2 * region : 0;
    return launch_forward(&g, nullptr, static_cast<char*>(workspace) + used, workspace_bytes > used ? workspace_bytes - used : 0, stream);
}

// The tuned backward kernels, in the three orders the entry point knows:
//   two launches     dV and dK workgroups side by side (the dK ones recompute S, dP and dS), then the query-tile
//                    kernel: eight matrix products, no workspace;
//   three launches   dV workgroups, the query-tile kernel storing dS, dK workgroups that read dS back: six products.
//                    dS is the attn_bias gradient when that is asked for (the dV workgroups clear it beside their
//                    work), otherwise it goes into a workspace of that shape, [batch, heads, max_seq_len_q,
//                    max_seq_len_k] in the input type;
//   planes           the query-tile kernel storing dS and P, then a dV workgroup that reads P and a dK workgroup that
//                    reads dS per key tile: the five products of the formula, nothing computed twice; a workspace of
//                    twice that size (per query row and 32-key block the 32 dS values, then the 32 P values: a whole
//                    128-byte line per row and step).  With an attn_bias gradient the query-tile kernel clears it
//                    beside its work and the dK workgroups write the dS pieces they read into it.
// Rows of 16 bytes are needed for the planes (max_seq_len_k a multiple of 8, 16-byte aligned pointers).  Nothing in a
// workspace is cleared: the workgroups that read a plane read exactly the pieces the query-tile kernel wrote.
//
// Which order is taken follows an estimate of each order's time from what the host knows (batch, total rows, longest
// sequence allowed, heads, head-dim slot, mask, attn_bias gradient or not), three terms per launch:
//   products   (visible pairs + 400 per query row and head for the diagonal blocks, the fill and the drain of a tile)
//              x products of the launch x the rate measured for that kernel family and head-dim slot with the machine
//              full (us per 10^6 pairs and product, B128 H4 L1024: key-tile kernel 0.197 / 0.336 / 0.891 at slots 64 /
//              128 / 256, query-tile kernel and the key-tile kernels fed from planes 0.111 / 0.216 / 0.554); the pairs
//              are estimated as for lengths spread evenly between 2 x mean - max and max;
//   planes     bytes written or read by the launch beyond its operands (dS 2 bytes per pair, dS and P 4, attn_bias 2, its
//              gradient 2 and the clearing of the whole gradient) / 10 TB/s for the part of them within 120 MB, which stays
//              in the memory-side cache between the launches, / 4.5 TB/s beyond (B128 H4 L1024: 537 MB of dS stored in
//              125 us, 1.07 GB of dS and P in 236 us);
//   tail       a launch lasts at least as long as its longest workgroup: (longest row / 32) steps (x query heads per K/V
//              head for key tiles) x (0.3 us + 0.2 / 0.33 / 0.7 us per product of the workgroup).
// A launch costs the larger of (products + planes) and tail, plus 2 us.  Checked on 34 shapes that none of the constants
// was taken from (examples/hstu_bwd_order_sweep.py): the order picked is within 10 % of the fastest on 33 of them; with an
// attn_bias gradient, on the 12 shapes of that example's set "bias", from which the slow-down of the variants that read
// attn_bias (1.25) and the charge for the gradient's second writing in the planes order were taken.
// Also tried, not kept: the dV workgroups on a second stream beside the query-tile kernel (C2 143 -> 149 us), and the
// query-tile kernel first with dV and dK-from-dS workgroups in one launch behind it (C2 160 us).
// HSTU_MI355_BWD_HANDOFF in the environment overrides the rule: 0 = two launches, 1 = three wherever possible,
// 2 = planes wherever possible.
enum BwdOrder { kTwoLaunches, kThreeLaunches, kPlanes };
struct BwdPlan {
    BwdOrder order;
    uint64_t workspace_bytes;  // what the order needs (0: none)
};

// The pair plane of the 16-bit backward kernels (dS and P of every (row, 32-key block) the query-tile kernel sweeps, one
// 128-byte line each; layout in hstu_bwd_kernel.hip.h): rows packed by global query row, and for a causal mask over equal
// offsets without context rows only the blocks at or below the diagonal -- sized from what the host knows without reading
// the offsets, total rows and the longest sequence allowed, with 32 rows of slack per sequence.
struct PairPlane {
    bool tri;
    int64_t head_lines;
    int64_t bytes;
    bool fits_32;  // one sequence's lines sit behind a 32-bit descriptor
};
static PairPlane pair_plane(const hstu_jagged_fwd_params* f)
{
    PairPlane pp;
    const int64_t batch = f->n_offsets - 1;
    const int64_t n_blk = (f->max_seq_len_k + 31) / 32;
    pp.tri = f->mask_type == HSTU_MASK_TRIL && f->num_context == nullptr && f->seq_offset_k == f->seq_offset_q &&
             f->total_k == f->total_q;
    const int64_t groups = ((f->max_seq_len_q < f->max_seq_len_k ? f->max_seq_len_q : f->max_seq_len_k) + 31) / 32;
    const int64_t pitch = hstu::pair_full_pitch_lines(f->max_seq_len_k);
    pp.head_lines = pp.tri ? ((f->total_q + 32 * batch) * (n_blk + 1) + 1) / 2 : f->total_q * pitch;
    pp.bytes = f->num_heads_q * pp.head_lines * 128;
    pp.fits_32 = (pp.tri ? 16 * groups * (groups + 1) : f->max_seq_len_q * pitch) * 128 < (1LL << 31);
    return pp;
}

// estimated microseconds of the three launch orders (see above)
struct BwdCost {
    double two, three, planes;
};
static BwdCost estimate_bwd(const hstu_jagged_fwd_params* f, bool bias_grad)
{
    static const double kRateKeyTile[3] = {0.197, 0.336, 0.891};  // us per 10^6 (pair x product), by head-dim slot
    static const double kRateOther[3] = {0.111, 0.216, 0.554};
    static const double kStepPerProduct[3] = {0.2, 0.33, 0.7};  // us per 32-key step of a workgroup
    const double kStepFixed = 0.3, kRowOverhead = 400.0, kCacheBytes = 120e6, kCachedBw = 10.0e6, kMemoryBw = 4.5e6;  // (bytes per us)
    const double kBiasSlowdown = 1.25;  // the variants that add attn_bias to the scores: fewer workgroups per CU
    const int64_t dmax = f->head_dim_qk > f->head_dim_v ? f->head_dim_qk : f->head_dim_v;
    const int slot = dmax <= 64 ? 0 : (dmax <= 128 ? 1 : 2);
    const double batch = static_cast<double>(f->n_offsets - 1), heads = static_cast<double>(f->num_heads_q);
    const double mean_q = static_cast<double>(f->total_q) / batch, mean_k = static_cast<double>(f->total_k) / batch;
    // max_seq_len is a bound, and callers often pass a configuration constant far above their sequences: lengths spread
    // evenly up to a longest one have a mean of half of it, so twice the mean stands in for a bound beyond that (a batch
    // of 32 sequences of 256..1024 rows under max_seq_len 8192 is then priced like the same batch under 1024: planes,
    // 174 -> 117 us, where the bound priced every order by one 8192-row tail and picked the two launches)
    const double max_q = std::max(mean_q, std::min(static_cast<double>(f->max_seq_len_q), 2.0 * mean_q));
    const double max_k = std::max(mean_k, std::min(static_cast<double>(f->max_seq_len_k), 2.0 * mean_k));
    const bool causal = f->mask_type == HSTU_MASK_TRIL;
    // sum over the sequences of (query rows x keys)
    double area = batch * (mean_q * mean_k + (max_q > mean_q && max_k > mean_k ? (max_q - mean_q) * (max_k - mean_k) / 3.0 : 0.0));
    area = std::min(area, static_cast<double>(f->total_q) * max_k);
    const double pairs = heads * area * (causal ? 0.5 : 1.0);
    const double mpairs = (pairs + (causal ? 1.0 : 0.4) * kRowOverhead * static_cast<double>(f->total_q) * heads) * 1e-6;
    const double ratio = static_cast<double>(f->num_heads_q / f->num_heads_k);
    const double dense = batch * heads * static_cast<double>(f->max_seq_len_q) * static_cast<double>(f->max_seq_len_k) * 2.0;  // the attn_bias gradient, cleared whole
    const double bias = bias_grad ? 2.0 * pairs : 0.0;         // attn_bias as read by a launch that computes scores
    auto launch = [&](int products, const double* rate, int products_per_wg, double bytes, bool key_tiles, bool scores) {
        const double cached = bytes > kCacheBytes ? kCacheBytes / bytes : 1.0;
        const double slow = (scores && bias_grad) ? kBiasSlowdown : 1.0;
        const double work = mpairs * products * rate[slot] * slow + bytes * (cached / kCachedBw + (1.0 - cached) / kMemoryBw);
        const double steps = (key_tiles ? max_q * ratio : max_k) / 32.0;
        const double tail = steps * (kStepFixed + products_per_wg * kStepPerProduct[slot]) * slow;
        return std::max(work, tail) + 2.0;
    };
    BwdCost c;
    if (!bias_grad) {
        c.two = launch(4, kRateKeyTile, 4, 0.0, true, true) + launch(3, kRateOther, 3, 0.0, false, true);
        c.three = launch(2, kRateKeyTile, 2, 0.0, true, true) + launch(3, kRateOther, 3, 2.0 * pairs, false, true) +
                  launch(1, kRateOther, 1, 2.0 * pairs, true, false);
        c.planes = launch(3, kRateOther, 3, 4.0 * pairs, false, true) + launch(2, kRateOther, 1, 4.0 * pairs, true, false);
    } else {
        // (the gradient is cleared beside the first launch's work and written by the query-tile kernel, or, in the planes
        // order, by the dK workgroups from the dS pieces they read)
        c.two = launch(4, kRateKeyTile, 4, bias + dense, true, true) + launch(3, kRateOther, 3, bias + 2.0 * pairs, false, true);
        c.three = launch(2, kRateKeyTile, 2, bias + dense, true, true) + launch(3, kRateOther, 3, bias + 2.0 * pairs, false, true) +
                  launch(1, kRateOther, 1, 2.0 * pairs, true, false);
        // (... in 16-byte pieces over lines cleared just before: charged as half the gradient once more, from memory)
        c.planes = launch(3, kRateOther, 3, bias + 4.0 * pairs + dense, false, true) + launch(2, kRateOther, 1, 6.0 * pairs, true, false) +
                   0.5 * dense / kMemoryBw;
    }
    return c;
}

static BwdPlan plan_bwd(const hstu_jagged_bwd_params* p, const BwdVariant* var)
{
    const hstu_jagged_fwd_params* f = &p->fwd;
    const BwdPlan two = {kTwoLaunches, 0};
    const int forced = switches().bwd_handoff;
    if (forced == 0 || f->total_q == 0 || f->total_k == 0) {
        return two;
    }
    if (f->dtype == HSTU_DT_FP32) {
        // the fp32 kernels know two orders: everything computed where it is used (7 products), or dS and P stored by the
        // query-tile kernel in fp32 and read back by the key-tile kernel (5 products, 16 bytes of traffic per pair).
        // The second is ahead wherever it was measured (recomputing -> planes): B16 H4 L100..1024 d32 245 -> 200 us,
        // d64 382 -> 264 us, d128 595 -> 439 us; B32 H8 L1024 d64 1557 -> 1344 us, d128 2899 -> 2233 us; B4 H4 d128
        // L300..700 405 -> 286 us; B2 H4 d128 L8192 4841 -> 4519 us -- the fp32 matrix instruction is slow enough for
        // a product to cost more than its operands' trip through memory.  Taken whenever the workspace is within the limit.
        if (var->dq_ds_p == nullptr) {
            return two;
        }
        const int64_t cap = workspace_cap_mb();
        const int64_t row = 64 * ((f->max_seq_len_k + 31) / 32);
        const int64_t bytes = (f->n_offsets - 1) * f->num_heads_q * f->max_seq_len_q * row * 4;
        const bool fits = f->max_seq_len_q * row * 4 < (1LL << 31) && bytes <= cap * (1LL << 20);
        return fits ? BwdPlan{kPlanes, static_cast<uint64_t>(bytes)} : two;
    }
    // Rows of the [max_q][max_k] tensors -- attn_bias, custom mask, the attn_bias gradient, a dense dS plane -- are read
    // and written by the key-tile kernels in pieces of 8 keys: one 16-byte access when max_seq_len_k is a multiple of 8,
    // two 8-byte ones when it is a multiple of 4; otherwise the call runs in two launches that take such rows element by
    // element.  The pair plane has a layout of its own: a call with none of those tensors can take the planes order
    // whatever max_seq_len_k is (max_seq_len 1004 instead of 1024 must not cost the two-launch order's 7 products).
    const bool rows8 = f->max_seq_len_k % 4 == 0;
    const bool no_bias_tensors = f->attn_bias == nullptr && f->mask == nullptr && p->grad_attn_bias == nullptr;
    if (var->dk_from_ds == nullptr || (!rows8 && !no_bias_tensors)) {
        return two;
    }
    const int64_t batch = f->n_offsets - 1;
    // (one sequence's part of a plane sits behind a 32-bit descriptor)
    if (f->max_seq_len_q * f->max_seq_len_k * 2 >= (1LL << 31)) {
        return two;
    }
    const bool bias_grad = p->grad_attn_bias != nullptr;
    const PairPlane pp = pair_plane(f);
    const int64_t dmax = f->head_dim_qk > f->head_dim_v ? f->head_dim_qk : f->head_dim_v;
    const int64_t cap_small = workspace_cap_mb() * (1LL << 20);
    const int64_t cap = workspace_cap_mb(dmax > 128) * (1LL << 20);
    // with an attn_bias gradient dS goes through the gradient itself in the three-launch order: no workspace
    const int64_t ds_plane = bias_grad ? 0 : batch * f->num_heads_q * f->max_seq_len_q * f->max_seq_len_k * 2;
    const bool three_fits = rows8 && ds_plane <= cap;
    const bool planes_fit = pp.fits_32 && pp.bytes <= cap && (!bias_grad || var->dv_dk_from_planes_drab != nullptr);
    const BwdPlan three = {kThreeLaunches, static_cast<uint64_t>(ds_plane)};
    const BwdPlan planes = {kPlanes, static_cast<uint64_t>(pp.bytes)};
    if (forced == 2) {
        return planes_fit ? planes : (three_fits ? three : two);
    }
    if (forced == 1) {
        return three_fits ? three : two;
    }
    const BwdCost cost = estimate_bwd(f, bias_grad);
    // the best order within the small limit, then the best of all: more than the small limit only for a tenth of the time
    BwdPlan best = two, best_small = two;
    double best_us = cost.two, best_small_us = cost.two;
    auto consider = [&](bool fits, const BwdPlan& plan, double us) {
        if (fits && us < best_us) {
            best = plan;
            best_us = us;
        }
        if (fits && static_cast<int64_t>(plan.workspace_bytes) <= cap_small && us < best_small_us) {
            best_small = plan;
            best_small_us = us;
        }
    };
    consider(three_fits, three, cost.three);
    consider(planes_fit, planes, cost.planes);
    if (static_cast<int64_t>(best.workspace_bytes) > cap_small && best_us > 0.9 * best_small_us) {
        return best_small;
    }
    return best;
}

// The query-tile kernel with 64-row tiles (hstu_bwd_dq_short_kernel.hip.h) where it is the faster one: 16-bit inputs at
// the head-dim slot 128 without bias or custom mask, in launches whose 128-row tiles would leave compute units idle
// (at most one (128-row tile, sequence, head) slot per compute unit: measured 9 to 16 % off the whole backward at
// 4 x 1024 to 16 x 512 rows with 4 heads, level at 1.5 slots per unit, 4 to 9 % slower from 2 slots on, where its
// 16-row matrix instructions cost more than the finer tiles bring).  HSTU_MI355_SHORT=0 / 1 overrides the rule.
static const hstu::DqShortVariant* dq_short_variant(const hstu_jagged_bwd_params* p, const BwdVariant* var)
{
    const hstu_jagged_fwd_params* f = &p->fwd;
    const int64_t dmax = f->head_dim_qk > f->head_dim_v ? f->head_dim_qk : f->head_dim_v;
    if ((f->dtype != HSTU_DT_BF16 && f->dtype != HSTU_DT_FP16) || f->attn_bias != nullptr || f->mask_type == HSTU_MASK_CUSTOM ||
        dmax <= 64 || dmax > 128 || f->head_dim_qk % 8 != 0 || is_generic_bwd(var) || var->dq_ds_p == nullptr) {
        return nullptr;
    }
    const int forced = switches().short_lists;
    if (forced == 0) {
        return nullptr;
    }
    if (forced != 1) {
        int cus = 0;
        const int64_t slots = ((f->max_seq_len_q + 127) / 128) * (f->n_offsets - 1) * f->num_heads_q;
        if (compute_units(&cus) != HSTU_OK || slots > cus) {
            return nullptr;
        }
    }
    return &hstu::bwd_variants_dq_short()[f->dtype == HSTU_DT_BF16 ? 0 : 1];
}
// grid of that kernel: one workgroup per (64-row tile, K/V pair padded to a multiple of 8, query head of the pair)
static int64_t dq_short_grid(const hstu::BwdArgs& a)
{
    const int64_t pairs_pad = (static_cast<int64_t>(a.n_batch) * a.n_heads_k + 7) & ~static_cast<int64_t>(7);
    return ((a.max_q + hstu::kDqShortRows - 1) / hstu::kDqShortRows) * pairs_pad * a.head_ratio;
}

// The whole backward in one launch for batches of tiny sequences (hstu_bwd_tiny_kernel.hip.h): 16-bit inputs with head
// dims up to 256 in multiples of 8, no bias (nor its gradient), no custom mask, no sequence longer than 32 rows or keys,
// every tensor on a 16-byte boundary.  No workspace.  Batch 2048 x 2 heads x 32 rows at head dim 256: 221 us on the tuned
// kernels (a 128-row workgroup per item in each of two launches).  HSTU_MI355_SHORT=0 switches it off.
static const hstu::BwdTinyVariant* bwd_tiny_variant(const hstu_jagged_bwd_params* p)
{
    const hstu_jagged_fwd_params* f = &p->fwd;
    const int64_t dmax = f->head_dim_qk > f->head_dim_v ? f->head_dim_qk : f->head_dim_v;
    const uintptr_t ptrs = reinterpret_cast<uintptr_t>(f->q) | reinterpret_cast<uintptr_t>(f->k) | reinterpret_cast<uintptr_t>(f->v) |
                           reinterpret_cast<uintptr_t>(p->grad) | reinterpret_cast<uintptr_t>(p->grad_q) |
                           reinterpret_cast<uintptr_t>(p->grad_k) | reinterpret_cast<uintptr_t>(p->grad_v);
    if ((f->dtype != HSTU_DT_BF16 && f->dtype != HSTU_DT_FP16) || f->attn_bias != nullptr || p->grad_attn_bias != nullptr ||
        f->mask_type == HSTU_MASK_CUSTOM || dmax > 256 || f->head_dim_qk % 8 != 0 || f->head_dim_v % 8 != 0 || ptrs % 16 != 0 ||
        f->max_seq_len_q > hstu::kTinyRows || f->max_seq_len_k > hstu::kTinyRows || f->n_offsets < 2 ||
        (f->n_offsets - 1) * f->num_heads_k > 0x7fffffffLL || switches().short_lists == 0 || switches().generic_backward == 1) {
        return nullptr;
    }
    return &hstu::bwd_variants_tiny()[f->dtype == HSTU_DT_BF16 ? 0 : 1][dmax <= 128 ? 0 : 1];
}

// The whole backward in one launch for sequences of few query rows (hstu_bwd_few_rows_kernel.hip.h): 16-bit inputs with
// head dims up to 128 in multiples of 8, no bias (nor its gradient), no custom mask, no sequence of more than 64 query rows
// (keys: any number), as many K/V heads as query heads, every tensor on a 16-byte boundary.  No workspace; K and V are
// read once.  HSTU_MI355_SHORT=0 switches it off.
static const hstu::BwdTinyVariant* bwd_few_rows_variant(const hstu_jagged_bwd_params* p)
{
    const hstu_jagged_fwd_params* f = &p->fwd;
    const int64_t dmax = f->head_dim_qk > f->head_dim_v ? f->head_dim_qk : f->head_dim_v;
    const uintptr_t ptrs = reinterpret_cast<uintptr_t>(f->q) | reinterpret_cast<uintptr_t>(f->k) | reinterpret_cast<uintptr_t>(f->v) |
                           reinterpret_cast<uintptr_t>(p->grad) | reinterpret_cast<uintptr_t>(p->grad_q) |
                           reinterpret_cast<uintptr_t>(p->grad_k) | reinterpret_cast<uintptr_t>(p->grad_v);
    const int64_t span_k = f->max_seq_len_k * f->num_heads_k * dmax * 2;
    if ((f->dtype != HSTU_DT_BF16 && f->dtype != HSTU_DT_FP16) || f->attn_bias != nullptr || p->grad_attn_bias != nullptr ||
        f->mask_type == HSTU_MASK_CUSTOM || dmax > 128 || f->head_dim_qk % 8 != 0 || f->head_dim_v % 8 != 0 || ptrs % 16 != 0 ||
        f->max_seq_len_q > hstu::kFewRows || f->num_heads_q != f->num_heads_k || f->n_offsets < 2 || span_k >= (1LL << 30) ||
        (f->n_offsets - 1) * f->num_heads_k > 0x7fffffffLL || switches().short_lists == 0 || switches().generic_backward == 1) {
        return nullptr;
    }
    return &hstu::bwd_variants_few_rows()[f->dtype == HSTU_DT_BF16 ? 0 : 1][dmax <= 64 ? 0 : 1];
}
// the one-launch kernels: tiny sequences first (it takes grouped heads and head dims up to 256), then few query rows
static const hstu::BwdTinyVariant* bwd_one_launch_variant(const hstu_jagged_bwd_params* p, unsigned* threads)
{
    if (const hstu::BwdTinyVariant* const tv = bwd_tiny_variant(p)) {
        *threads = hstu::kTinyThreads;
        return tv;
    }
    *threads = hstu::kFewRowsThreads;
    return bwd_few_rows_variant(p);
}

// Head dims above 256 on the matrix pipe: 16-bit inputs whose head dims are multiples of 16 run as two windows per head
// on the kernels of the slot 256 (heads taken as 2 x heads of half the dims): the query-tile kernel over the first window
// (S and dP in fp32 to a partial plane), over the second (adds them up: dS and P to the pair plane, dQ of the second
// window), once more for dQ of the first window from the stored dS, then the dV-from-P / dK-from-dS workgroups of all
// windows.  Needs its workspace (partial plane: 256 bytes per query row, 32-key block and head; pair plane as in the planes
// order): a call without it, or one whose planes pass the limit, runs on the generic kernels.  B8 H4 d512 L100..1024:
// 37 ms on the generic kernels.  HSTU_MI355_GENERIC_BACKWARD=1 keeps the generic kernels.
struct WindowPlan {
    const BwdVariant* var;  // nullptr: not this path
    PairPlane pair;
    uint64_t partial_bytes;
    uint64_t workspace_bytes;
};
static WindowPlan plan_windows(const hstu_jagged_bwd_params* p)
{
    WindowPlan w;
    memset(&w, 0, sizeof(w));
    const hstu_jagged_fwd_params* f = &p->fwd;
    const int64_t dmax = f->head_dim_qk > f->head_dim_v ? f->head_dim_qk : f->head_dim_v;
    if ((f->dtype != HSTU_DT_BF16 && f->dtype != HSTU_DT_FP16) || dmax <= 256 || dmax > 512 || f->head_dim_qk % 16 != 0 ||
        f->head_dim_v % 16 != 0 || switches().generic_backward == 1 || f->total_q == 0 || f->total_k == 0) {
        return w;
    }
    // (rows of attn_bias, custom mask and the gradient are read and written in pieces of 8 or 16 bytes: see plan_bwd)
    const bool no_bias_tensors = f->attn_bias == nullptr && f->mask == nullptr && p->grad_attn_bias == nullptr;
    if (f->max_seq_len_k % 4 != 0 && !no_bias_tensors) {
        return w;
    }
    // (16-byte rows of the planes and of the attn_bias tensors, spans behind 32-bit descriptors)
    const uintptr_t ptrs = reinterpret_cast<uintptr_t>(f->attn_bias) | reinterpret_cast<uintptr_t>(f->mask) |
                           reinterpret_cast<uintptr_t>(p->grad_attn_bias);
    const int64_t span_q = f->max_seq_len_q * f->num_heads_q * dmax * 2;
    const int64_t span_k = f->max_seq_len_k * f->num_heads_k * dmax * 2;
    const int64_t span_b = f->max_seq_len_q * f->max_seq_len_k * 2;
    if (ptrs % 16 != 0 || span_q >= (1LL << 30) || span_k >= (1LL << 30) || span_b >= (1LL << 31)) {
        return w;
    }
    w.pair = pair_plane(f);
    const int64_t n_blk = (f->max_seq_len_k + 31) / 32;
    w.partial_bytes = static_cast<uint64_t>(f->num_heads_q * f->total_q * n_blk * 256);
    w.workspace_bytes = static_cast<uint64_t>(w.pair.bytes) + w.partial_bytes;
    // (without the workspace these head dims run on the generic kernels: the larger limit)
    if (!w.pair.fits_32 || w.workspace_bytes > static_cast<uint64_t>(workspace_cap_mb(true)) * (1ULL << 20)) {
        return w;
    }
    const auto* table = f->dtype == HSTU_DT_BF16 ? hstu::bwd_variants_bf16() : hstu::bwd_variants_f16();
    w.var = &table[f->attn_bias != nullptr ? 1 : 0][f->mask_type == HSTU_MASK_CUSTOM ? 1 : 0][2];
    return w;
}

HSTU_API int hstu_jagged_bwd_workspace_size(const hstu_jagged_bwd_params* params, uint64_t* workspace_bytes)
{
    if (workspace_bytes == nullptr) {
        return fail(HSTU_ERR_NULLPTR, "workspace_bytes is NULL");
    }
    *workspace_bytes = 0;
    const int rc = validate_bwd(params);
    if (rc != HSTU_OK) {
        return rc;
    }
    const BwdVariant* var = select_bwd(params);
    if (var == nullptr) {
        return HSTU_ERR_UNSUPPORTED;
    }
    unsigned one_launch_threads = 0;
    if (bwd_one_launch_variant(params, &one_launch_threads) != nullptr) {
        return HSTU_OK;
    }
    const WindowPlan windows = plan_windows(params);
    *workspace_bytes = windows.var != nullptr ? windows.workspace_bytes : plan_bwd(params, var).workspace_bytes;
    return HSTU_OK;
}

HSTU_API int hstu_jagged_bwd(const hstu_jagged_bwd_params* p, void* workspace, uint64_t workspace_bytes, void* stream)
{
    const int rc = validate_bwd(p);
    if (rc != HSTU_OK) {
        return rc;
    }
    const BwdVariant* var = select_bwd(p);
    if (var == nullptr) {
        return HSTU_ERR_UNSUPPORTED;
    }
    const hstu_jagged_fwd_params* f = &p->fwd;
    // the attn_bias gradient is written in full: cleared by the key-tile kernel beside its work (or by a fill of
    // its own when that kernel has nothing to run on), then written by the query-tile kernel where its tiles sweep
    const int64_t es = f->dtype == HSTU_DT_FP32 ? 4 : 2;
    const int64_t drab_bytes = (p->grad_attn_bias != nullptr)
                                   ? (f->n_offsets - 1) * f->num_heads_q * f->max_seq_len_q * f->max_seq_len_k * es
                                   : 0;
    if (f->total_q == 0 && f->total_k == 0) {
        if (drab_bytes > 0) {
            launch_clear(p->grad_attn_bias, drab_bytes, stream);
        }
        return HSTU_OK;
    }
    hstu::BwdArgs a;
    memset(&a, 0, sizeof(a));
    a.win = 1;
    a.win_only = -1;
    a.q = f->q;
    a.k = f->k;
    a.v = f->v;
    a.grad = p->grad;
    a.rab = f->attn_bias;
    a.mask = (f->mask_type == HSTU_MASK_CUSTOM) ? f->mask : nullptr;
    a.dq = p->grad_q;
    a.dk = p->grad_k;
    a.dv = p->grad_v;
    a.drab = p->grad_attn_bias;
    a.grad_vec_ok = (f->head_dim_qk % 8 == 0 && f->head_dim_v % 8 == 0 && reinterpret_cast<uintptr_t>(p->grad_q) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(p->grad_k) % 16 == 0 && reinterpret_cast<uintptr_t>(p->grad_v) % 16 == 0)
                        ? 1
                        : 0;
    a.offs_q = f->seq_offset_q;
    a.offs_k = f->seq_offset_k;
    a.num_ctx = f->num_context;
    a.num_tgt = f->num_target;
    a.total_q = f->total_q;
    a.total_k = f->total_k;
    a.n_batch = static_cast<int>(f->n_offsets - 1);
    a.n_heads_q = static_cast<int>(f->num_heads_q);
    a.n_heads_k = static_cast<int>(f->num_heads_k);
    a.head_ratio = a.n_heads_q / a.n_heads_k;
    a.d_qk = static_cast<int>(f->head_dim_qk);
    a.d_v = static_cast<int>(f->head_dim_v);
    a.max_q = static_cast<int>(f->max_seq_len_q);
    a.max_k = static_cast<int>(f->max_seq_len_k);
    a.mask_type = static_cast<int>(f->mask_type);
    a.target_group = static_cast<int>(f->target_group_size);
    a.idx64 = (f->index_dtype == HSTU_IDX_I64) ? 1 : 0;
    a.n_qtiles = (a.max_q + hstu::kBlockM - 1) / hstu::kBlockM;
    a.n_ktiles = (a.max_k + hstu::kBlockM - 1) / hstu::kBlockM;
    a.bias_vec_ok = (reinterpret_cast<uintptr_t>(f->attn_bias) % 8 == 0 && reinterpret_cast<uintptr_t>(f->mask) % 8 == 0 &&
                     reinterpret_cast<uintptr_t>(p->grad_attn_bias) % 8 == 0 && f->max_seq_len_k % 4 == 0)
                        ? 1
                        : 0;
    if (a.bias_vec_ok != 0 && reinterpret_cast<uintptr_t>(f->attn_bias) % 16 == 0 && reinterpret_cast<uintptr_t>(f->mask) % 16 == 0 &&
        reinterpret_cast<uintptr_t>(p->grad_attn_bias) % 16 == 0 && f->max_seq_len_k % 8 == 0) {
        a.bias_vec_ok = 2;  // 16-byte aligned rows: the key-tile kernel reads rab / mask rows 16 bytes per lane
    }
    if (f->dtype == HSTU_DT_FP32) {  // four fp32 elements = 16 bytes
        a.bias_vec_ok = (reinterpret_cast<uintptr_t>(f->attn_bias) % 16 == 0 && reinterpret_cast<uintptr_t>(f->mask) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(p->grad_attn_bias) % 16 == 0 && f->max_seq_len_k % 4 == 0)
                            ? 1
                            : 0;
    }
    a.alpha = static_cast<float>(f->alpha);
    a.scale = static_cast<float>((f->silu_scale == 0.0) ? 1.0 / static_cast<double>(f->max_seq_len_q) : f->silu_scale);

    unsigned one_launch_threads = 0;
    if (const hstu::BwdTinyVariant* const tv = bwd_one_launch_variant(p, &one_launch_threads)) {
        hipLaunchKernelGGL(tv->kernel, dim3(static_cast<unsigned>(a.n_batch * a.n_heads_k)), dim3(one_launch_threads), 0,
                           static_cast<hipStream_t>(stream), a);
        const hipError_t err_tiny = hipGetLastError();
        if (err_tiny != hipSuccess) {
            return fail(HSTU_ERR_RUNTIME, "launch of %s failed: %s", tv->name, hipGetErrorString(err_tiny));
        }
        return HSTU_OK;
    }
    const WindowPlan windows = plan_windows(p);
    if (windows.var != nullptr && usable_workspace(workspace, workspace_bytes, windows.workspace_bytes) &&
        reinterpret_cast<uintptr_t>(workspace) % 16 == 0 && a.grad_vec_ok != 0) {
        const BwdVariant* const wv = windows.var;
        hstu::BwdArgs w = a;
        w.win = 2;
        w.d_qk = a.d_qk / 2;
        w.d_v = a.d_v / 2;
        w.n_heads_q = 2 * a.n_heads_q;
        w.n_heads_k = 2 * a.n_heads_k;
        w.bias_vec_ok = f->max_seq_len_k % 8 == 0 ? 2 : 1;  // (pointers are 16-byte aligned here; rows of 16 or of 8 bytes)
        w.p_plane = workspace;
        w.plane_head_lines = windows.pair.head_lines;
        w.plane_tri = windows.pair.tri ? 1 : 0;
        w.partial = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + windows.pair.bytes);
        const int64_t grid_q = static_cast<int64_t>(a.n_qtiles) * a.n_batch * a.n_heads_q;  // (real heads: one window per launch)
        const int64_t kv_slots = static_cast<int64_t>(a.n_ktiles) * a.n_batch * w.n_heads_k;
        const int64_t grid_kv = 16 * ((kv_slots + 7) / 8);
        if (grid_kv > 0x7fffffffLL || grid_q > 0x7fffffffLL) {
            return fail(HSTU_ERR_INVALID, "grid out of range");
        }
        w.win_only = 0;
        hipLaunchKernelGGL(wv->dq_win_first, dim3(static_cast<unsigned>(grid_q)), dim3(256), 0, static_cast<hipStream_t>(stream), w);
        w.win_only = 1;
        w.drab_clear_bytes = drab_bytes;
        hipLaunchKernelGGL(wv->dq_win_second_ds_p, dim3(static_cast<unsigned>(grid_q)), dim3(256), 0, static_cast<hipStream_t>(stream), w);
        w.drab_clear_bytes = 0;
        w.win_only = 0;
        hipLaunchKernelGGL(wv->dq_win_from_plane, dim3(static_cast<unsigned>(grid_q)), dim3(256), 0, static_cast<hipStream_t>(stream), w);
        w.win_only = -1;
        hipLaunchKernelGGL(p->grad_attn_bias != nullptr ? wv->dv_dk_from_planes_drab : wv->dv_dk_from_planes,
                           dim3(static_cast<unsigned>(grid_kv)), dim3(hstu::kDkvThreads), 0, static_cast<hipStream_t>(stream), w);
        const hipError_t err_w = hipGetLastError();
        if (err_w != hipSuccess) {
            return fail(HSTU_ERR_RUNTIME, "launch of %s (two windows) failed: %s", wv->name, hipGetErrorString(err_w));
        }
        return HSTU_OK;
    }
    const bool generic = is_generic_bwd(var);
    const BwdPlan plan = plan_bwd(p, var);
    const hstu::DqShortVariant* const dq_short = generic ? nullptr : dq_short_variant(p, var);
    // The order of the slots in the grids of the tuned kernels (slot_of in hstu_bwd_kernel.hip.h): pair after pair, on one
    // XCD each, where level after level would have every resident workgroup stream another pair's rows from memory --
    // K, V, Q and dO of the call together beyond the 256 MB memory-side cache, at the head-dim slots that run two workgroups
    // per CU (at the slot 256 a step takes twice as long per byte it streams, and memory keeps up: 96 x 2 heads of 3072 rows
    // 6.59 ms level after level, 6.90 ms pair after pair) -- and the launch is long enough for the pairs left at its end not to
    // matter (8 tiles per workgroup that fits the machine, by the mean length).  Measured, bf16 d 128, 4 heads: 128 x 7621 rows
    // 40.5 -> 32.9 ms, 64 x 4096 rows 5.83 -> 5.04 ms, 64 x 1024..4096 rows 2.92 -> 2.58 ms, 256 x 1024 rows level.
    if (!generic && dq_short == nullptr) {
        int cus = 0;
        if (compute_units(&cus) != HSTU_OK) {
            return HSTU_ERR_RUNTIME;
        }
        const int64_t row_bytes = (f->head_dim_qk + f->head_dim_v) * es;
        const int64_t streamed = f->total_k * f->num_heads_k * row_bytes + f->total_q * f->num_heads_q * row_bytes;
        const int64_t tiles = (f->total_q / hstu::kBlockM) * f->num_heads_q;
        const int64_t dmax = f->head_dim_qk > f->head_dim_v ? f->head_dim_qk : f->head_dim_v;
        // (the slot 256: jagged batches only -- 64 x 4 heads of 1024..4096 rows 8.87 -> 7.91 ms, 256 x 4 of 256..1024 rows 1.93 -> 1.68 ms)
        const bool jagged = 10 * f->total_q <= 7 * (f->n_offsets - 1) * f->max_seq_len_q;
        // (jagged batches from half of that on: 16 x 8 heads of 1024..4096 rows 1.35 -> 1.19 ms, 64 x 4 of 512..2048 rows 813 -> 774 us;
        // equally long sequences lose there: 32 x 8 of 1024 rows 436 -> 512 us)
        const bool long_launch = ((dmax <= 128 || jagged) && streamed >= (512LL << 20) && tiles >= 16LL * cus) ||
                                 (dmax <= 128 && jagged && streamed >= (256LL << 20) && tiles >= 8LL * cus);
        const int forced = switches().bwd_pair_major;
        a.pair_major = forced >= 0 ? forced : (long_launch ? 1 : 0);
    }
    const int64_t pairs_q = static_cast<int64_t>(a.n_batch) * a.n_heads_q, pairs_k = static_cast<int64_t>(a.n_batch) * a.n_heads_k;
    // the tuned key-tile kernel runs a dV and a dK workgroup per tile, the generic one a workgroup per tile
    const int64_t n_kv_slots = static_cast<int64_t>(a.n_ktiles) * (a.pair_major ? 8 * ((pairs_k + 7) / 8) : pairs_k);
    // (with both roles in a launch: groups of 8 dV workgroups followed by their 8 dK workgroups, whole groups)
    const int64_t grid_kv = generic ? n_kv_slots : 16 * ((n_kv_slots + 7) / 8);
    const int64_t grid_q = static_cast<int64_t>(a.n_qtiles) * (a.pair_major ? 8 * ((pairs_q + 7) / 8) : pairs_q);
    if (grid_kv > 0x7fffffffLL || grid_q > 0x7fffffffLL) {
        return fail(HSTU_ERR_INVALID, "grid out of range");
    }
    if (generic) {
        // the generic kernels write what they compute and nothing else: every output starts from zero
        launch_clear(p->grad_q, f->total_q * f->num_heads_q * f->head_dim_qk * es, stream);
        launch_clear(p->grad_k, f->total_k * f->num_heads_k * f->head_dim_qk * es, stream);
        launch_clear(p->grad_v, f->total_k * f->num_heads_k * f->head_dim_v * es, stream);
        if (drab_bytes > 0) {
            launch_clear(p->grad_attn_bias, drab_bytes, stream);
        }
        if (f->total_k > 0 && f->total_q > 0 && grid_kv > 0 && grid_q > 0) {
            if (plan.order == kPlanes && usable_workspace(workspace, workspace_bytes, plan.workspace_bytes) &&
                reinterpret_cast<uintptr_t>(workspace) % 16 == 0) {
                // (fp32) the query-tile kernel leaves dS and P in the workspace, the key-tile kernel reads them back
                a.p_plane = workspace;
                hipLaunchKernelGGL(var->dq_ds_p, dim3(static_cast<unsigned>(grid_q)), dim3(256), 0, static_cast<hipStream_t>(stream), a);
                hipLaunchKernelGGL(var->dv_dk_from_planes, dim3(static_cast<unsigned>(grid_kv)), dim3(256), 0,
                                   static_cast<hipStream_t>(stream), a);
            } else {
                hipLaunchKernelGGL(var->dkv, dim3(static_cast<unsigned>(grid_kv)), dim3(256), 0, static_cast<hipStream_t>(stream), a);
                hipLaunchKernelGGL(var->dq, dim3(static_cast<unsigned>(grid_q)), dim3(256), 0, static_cast<hipStream_t>(stream), a);
            }
        }
    } else if (f->total_k > 0 && grid_kv > 0 && f->total_q > 0 && grid_q > 0 && plan.order != kTwoLaunches &&
               (a.bias_vec_ok != 0 || (plan.order == kPlanes && f->attn_bias == nullptr && f->mask == nullptr && p->grad_attn_bias == nullptr)) &&
               (plan.workspace_bytes == 0 || (usable_workspace(workspace, workspace_bytes, plan.workspace_bytes) &&
                                              reinterpret_cast<uintptr_t>(workspace) % 16 == 0))) {
        if (p->grad_attn_bias == nullptr) {
            a.drab = workspace;
        }
        if (plan.order == kPlanes) {
            // the query-tile kernel with dS and P (clearing the attn_bias gradient beside its work when there is one),
            // then a dV-from-P and a dK-from-dS workgroup per key tile (the latter writing dS into that gradient)
            const PairPlane pp = pair_plane(f);
            a.p_plane = workspace;
            a.plane_head_lines = pp.head_lines;
            a.plane_tri = pp.tri ? 1 : 0;
            a.drab_clear_bytes = drab_bytes;
            if (dq_short != nullptr) {
                hipLaunchKernelGGL(dq_short->dq_ds_p, dim3(static_cast<unsigned>(dq_short_grid(a))), dim3(hstu::kDqShortThreads), 0,
                                   static_cast<hipStream_t>(stream), a);
            } else {
                hipLaunchKernelGGL(var->dq_ds_p, dim3(static_cast<unsigned>(grid_q)), dim3(256), 0, static_cast<hipStream_t>(stream), a);
            }
            a.drab_clear_bytes = 0;
            hipLaunchKernelGGL(p->grad_attn_bias != nullptr ? var->dv_dk_from_planes_drab : var->dv_dk_from_planes,
                               dim3(static_cast<unsigned>(grid_kv)), dim3(hstu::kDkvThreads), 0,
                               static_cast<hipStream_t>(stream), a);
            const hipError_t err2 = hipGetLastError();
            if (err2 != hipSuccess) {
                return fail(HSTU_ERR_RUNTIME, "launch of %s failed: %s", var->name, hipGetErrorString(err2));
            }
            return HSTU_OK;
        }
        // dV workgroups (which clear the attn_bias gradient beside their work), the query-tile kernel (which writes
        // dS into it, or into the workspace), dK workgroups (which read dS back)
        a.drab_clear_bytes = drab_bytes;
        hipLaunchKernelGGL(var->dv_only, dim3(static_cast<unsigned>(n_kv_slots)), dim3(hstu::kDkvThreads), 0,
                           static_cast<hipStream_t>(stream), a);
        a.drab_clear_bytes = 0;
        if (dq_short != nullptr && p->grad_attn_bias == nullptr && a.bias_vec_ok == 2) {  // (its dS pieces assume 16-byte rows)
            hipLaunchKernelGGL(dq_short->dq_ds, dim3(static_cast<unsigned>(dq_short_grid(a))), dim3(hstu::kDqShortThreads), 0,
                               static_cast<hipStream_t>(stream), a);
        } else {
            hipLaunchKernelGGL(var->dq_drab, dim3(static_cast<unsigned>(grid_q)), dim3(256), 0, static_cast<hipStream_t>(stream), a);
        }
        hipLaunchKernelGGL(var->dk_from_ds, dim3(static_cast<unsigned>(n_kv_slots)), dim3(hstu::kDkvThreads), 0,
                           static_cast<hipStream_t>(stream), a);
        const hipError_t err3 = hipGetLastError();
        if (err3 != hipSuccess) {
            return fail(HSTU_ERR_RUNTIME, "launch of %s failed: %s", var->name, hipGetErrorString(err3));
        }
        return HSTU_OK;
    } else if (f->total_k > 0 && grid_kv > 0) {
        a.drab_clear_bytes = drab_bytes;
        hipLaunchKernelGGL(var->dkv, dim3(static_cast<unsigned>(grid_kv)), dim3(hstu::kDkvThreads), 0,
                           static_cast<hipStream_t>(stream), a);
    } else if (drab_bytes > 0) {
        launch_clear(p->grad_attn_bias, drab_bytes, stream);
    }
    if (!generic && f->total_q > 0 && grid_q > 0) {
        if (dq_short != nullptr && p->grad_attn_bias == nullptr) {
            hipLaunchKernelGGL(dq_short->dq, dim3(static_cast<unsigned>(dq_short_grid(a))), dim3(hstu::kDqShortThreads), 0,
                               static_cast<hipStream_t>(stream), a);
        } else {
            hipLaunchKernelGGL(p->grad_attn_bias != nullptr ? var->dq_drab : var->dq, dim3(static_cast<unsigned>(grid_q)), dim3(256),
                               0, static_cast<hipStream_t>(stream), a);
        }
    }
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        return fail(HSTU_ERR_RUNTIME, "launch of %s failed: %s", var->name, hipGetErrorString(err));
    }
    return HSTU_OK;
}

HSTU_API int hstu_version(void) { return (0 << 16) | 1; }

HSTU_API const char* hstu_last_error(void) { return g_err; }

HSTU_API void hstu_reload_switches(void)
{
    switches();  // (so that the one-time read cannot come after this one)
    read_switches();
}

HSTU_API int hstu_jagged_fwd_workspace_size(const hstu_jagged_fwd_params* params, uint64_t* workspace_bytes)
{
    if (workspace_bytes == nullptr) {
        return fail(HSTU_ERR_NULLPTR, "workspace_bytes is NULL");
    }
    *workspace_bytes = 0;
    const int rc = validate(params);
    if (rc != HSTU_OK) {
        return rc;
    }
    const Variant* v = select(params);
    if (v == nullptr) {
        return HSTU_ERR_UNSUPPORTED;
    }
    // The tile schedule is derived inside the kernel from seq_offset.  Scratch is asked for by long lists (work
    // counters of the per-XCD queues) and by short ones (counters and room for the partial outputs of split items,
    // see split_workspace_bytes); a caller that brings less, or none, is served by the fixed schedule of the plain
    // list.  Without a usable device the answer is 0.
    *workspace_bytes = forward_workspace_bytes(v, params);
    return HSTU_OK;
}

HSTU_API const char* hstu_jagged_fwd_kernel_name(const hstu_jagged_fwd_params* params)
{
    if (validate(params) != HSTU_OK) {
        return nullptr;
    }
    const Variant* v = select(params);
    if (v == nullptr) {
        return nullptr;
    }
    // (given the workspace asked for; without a usable device the plain name is reported)
    unsigned one_item_threads = 0;
    if (const hstu::ShortVariant* const tv = one_item_variant(v, params, &one_item_threads)) {
        return tv->name;
    }
    if (const hstu::ShortVariant* const sv = short_variant(v, params)) {
        return sv->name;
    }
    if (takes_queue_variant(v, params, nullptr)) {
        return v->name_queues;
    }
    return may_take_split_variant(v, params, nullptr) ? v->name_split : v->name;
}

}  // extern "C"

namespace {

// the forward launch; `paged` (optional) makes it the paged variant, which the caller has checked to exist
int launch_forward(const hstu_jagged_fwd_params* p, const hstu_paged_fwd_params* paged, void* workspace,
                   uint64_t workspace_bytes, void* stream)
{
    const int rc = validate(p);
    if (rc != HSTU_OK) {
        return rc;
    }
    const Variant* var = select(p);
    if (var == nullptr) {
        return HSTU_ERR_UNSUPPORTED;
    }
    if (p->total_q == 0) {
        return HSTU_OK;
    }

    hstu::FwdArgs a;
    memset(&a, 0, sizeof(a));
    a.q = p->q;
    a.k = p->k;
    a.v = p->v;
    a.rab = p->attn_bias;
    a.mask = (p->mask_type == HSTU_MASK_CUSTOM) ? p->mask : nullptr;
    a.out = p->out;
    a.offs_q = p->seq_offset_q;
    a.offs_k = p->seq_offset_k;
    a.num_ctx = p->num_context;
    a.num_tgt = p->num_target;
    a.total_q = p->total_q;
    a.total_k = p->total_k;
    a.n_batch = static_cast<int>(p->n_offsets - 1);
    a.n_heads_q = static_cast<int>(p->num_heads_q);
    a.n_heads_k = static_cast<int>(p->num_heads_k);
    a.head_ratio = a.n_heads_q / a.n_heads_k;
    a.d_qk = static_cast<int>(p->head_dim_qk);
    a.d_v = static_cast<int>(p->head_dim_v);
    a.max_q = static_cast<int>(p->max_seq_len_q);
    a.max_k = static_cast<int>(p->max_seq_len_k);
    a.mask_type = static_cast<int>(p->mask_type);
    a.target_group = static_cast<int>(p->target_group_size);
    a.idx64 = (p->index_dtype == HSTU_IDX_I64) ? 1 : 0;
    a.n_qtiles = (a.max_q + hstu::kBlockM - 1) / hstu::kBlockM;
    a.bh = a.n_batch * a.n_heads_q;
    const uintptr_t vec_bytes = (p->dtype == HSTU_DT_FP32) ? 16 : (p->dtype == HSTU_DT_FP8_E4M3 ? 4 : 8);  // four elements
    const bool bias_aligned = (reinterpret_cast<uintptr_t>(p->attn_bias) % vec_bytes == 0) &&
                              (reinterpret_cast<uintptr_t>(p->mask) % vec_bytes == 0) && (p->max_seq_len_k % 4 == 0);
    a.bias_vec_ok = bias_aligned ? 1 : 0;
    a.out_vec_ok = (p->head_dim_v % 8 == 0 && reinterpret_cast<uintptr_t>(p->out) % 16 == 0) ? 1 : 0;
    if (bias_aligned && (p->dtype == HSTU_DT_BF16 || p->dtype == HSTU_DT_FP16) && reinterpret_cast<uintptr_t>(p->attn_bias) % 16 == 0 &&
        reinterpret_cast<uintptr_t>(p->mask) % 16 == 0 && p->max_seq_len_k % 8 == 0) {
        a.bias_vec_ok = 2;  // 16-byte row alignment: the 16-bit kernels read rab / mask rows 32 bytes per lane
    }
    const double scale = (p->silu_scale == 0.0) ? 1.0 / static_cast<double>(p->max_seq_len_q) : p->silu_scale;
    a.c_exp = static_cast<float>(-p->alpha * 1.4426950408889634);
    a.c_out = static_cast<float>(p->alpha * scale);
    a.alpha = static_cast<float>(p->alpha);
    a.silu_scale = static_cast<float>(scale);
    a.fp8_scaled_p = p->fp8_scaled_p != 0 ? 1 : 0;
    a.q_descale = p->q_descale;
    a.k_descale = p->k_descale;
    a.v_descale = p->v_descale;
    if (paged != nullptr) {
        a.kv_cache = paged->kv_cache;
        a.page_offsets = paged->page_offsets;
        a.page_ids = paged->page_ids;
        a.num_pages = paged->num_pages;
        a.n_page_ids = paged->n_page_ids;
        a.page_shift = paged->page_size == 32 ? 5 : paged->page_size == 64 ? 6 : paged->page_size == 128 ? 7 : 8;
    }

    int64_t n_blocks = static_cast<int64_t>(a.n_qtiles) * a.bh;  // one per (query tile, sequence, head) slot
    if (n_blocks <= 0 || n_blocks > 0x7fffffffLL) {
        return fail(HSTU_ERR_INVALID, "grid of %lld workgroups is out of range", (long long)n_blocks);
    }
    unsigned one_item_threads = 0;
    if (const hstu::ShortVariant* const tv = (paged == nullptr) ? one_item_variant(var, p, &one_item_threads) : nullptr) {
        // one workgroup per (sequence, query head)
        hipLaunchKernelGGL(tv->kernel, dim3(static_cast<unsigned>(a.bh)), dim3(one_item_threads), 0, static_cast<hipStream_t>(stream), a);
        const hipError_t err_tiny = hipGetLastError();
        if (err_tiny != hipSuccess) {
            return fail(HSTU_ERR_RUNTIME, "launch of %s failed: %s", tv->name, hipGetErrorString(err_tiny));
        }
        return HSTU_OK;
    }
    if (const hstu::ShortVariant* const sv =
            (paged == nullptr) ? short_variant(var, p, usable_workspace(workspace, workspace_bytes, kCounterBytes)) : nullptr) {
        // one workgroup per (query tile, K/V pair padded to a multiple of 8, query head of the pair) slot
        const int64_t pairs_pad = (static_cast<int64_t>(a.n_batch) * a.n_heads_k + 7) & ~static_cast<int64_t>(7);
        const int64_t slots = static_cast<int64_t>(a.n_qtiles) * pairs_pad * a.head_ratio;
        if (slots > (1LL << 22)) {
            return fail(HSTU_ERR_INVALID, "grid of %lld workgroups is out of range", (long long)slots);
        }
#ifdef HSTU_TIMELINE
        if (const char* const t = getenv("HSTU_TIMELINE_BUFFER")) {
            a.counters = reinterpret_cast<unsigned int*>(strtoull(t, nullptr, 0));  // development builds: where the workgroups leave their time stamps
        }
#endif
        hipLaunchKernelGGL(sv->kernel, dim3(static_cast<unsigned>(slots)), dim3(hstu::kShortThreads), 0,
                           static_cast<hipStream_t>(stream), a);
        const hipError_t err_short = hipGetLastError();
        if (err_short != hipSuccess) {
            return fail(HSTU_ERR_RUNTIME, "launch of %s failed: %s", sv->name, hipGetErrorString(err_short));
        }
        return HSTU_OK;
    }
    void (*kernel)(const hstu::FwdArgs) = var->kernel;
    if (var->persistent_wgs_per_cu > 0) {
        // persistent kernel: a fixed number of workgroups pulls the (at most n_blocks) work items
        int cus = 0;
        const int rc_cu = compute_units(&cus);
        if (rc_cu != HSTU_OK) {
            return rc_cu;
        }
        int64_t resident = static_cast<int64_t>(cus) * wgs_per_cu(var, p);
        // the variants that pull items from counters need the counter block at the head of the workspace; without
        // it every list runs on the plain variant's fixed schedule
        const bool have_counters = usable_workspace(workspace, workspace_bytes, kCounterBytes);
        if (have_counters && takes_queue_variant(var, p, &resident)) {
            kernel = var->kernel_queues;
            a.counters = static_cast<unsigned int*>(workspace);
        }
        n_blocks = n_blocks < resident ? n_blocks : resident;
        const uint64_t part_bytes = split_part_bytes(var);
        if (usable_workspace(workspace, workspace_bytes, kCounterBytes + 2 * part_bytes) && may_take_split_variant(var, p, nullptr)) {
            kernel = var->kernel_split;
            a.counters = static_cast<unsigned int*>(workspace);
            a.ws = reinterpret_cast<float*>(static_cast<char*>(workspace) + kCounterBytes);
            const uint64_t parts = (workspace_bytes - kCounterBytes) / part_bytes;
            a.ws_parts = static_cast<uint32_t>(parts < 0x7fffffffull ? parts : 0x7fffffffull);
            n_blocks = resident;  // the list may have more entries than items: all resident workgroups take part
        }
        if (paged != nullptr) {
            kernel = var->kernel_paged;  // (splits when it was given room above, otherwise not; the caller checked the block)
            a.counters = static_cast<unsigned int*>(workspace);
        }
        if (a.counters != nullptr) {
            launch_clear(a.counters, static_cast<int64_t>(kCounterBytes), stream);
        }
    }
    // (the kernel for head dims above 256 takes a workgroup per window of 256 output dims)
    const Variant* const wide0 = &hstu::fwd_variants_wide()[0][0][0];
    const unsigned out_windows = (var >= wide0 && var < wide0 + 8 && p->head_dim_v > 256) ? 2u : 1u;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(n_blocks), out_windows), dim3(static_cast<unsigned>(var->threads)), 0,
                       static_cast<hipStream_t>(stream), a);
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        return fail(HSTU_ERR_RUNTIME, "launch of %s failed: %s", var->name, hipGetErrorString(err));
    }
    return HSTU_OK;
}

}  // namespace

namespace {

// device address of `scratch` on the current GPU, looked up once per device (with that device current); the array's
// name is a host-side stand-in and never goes to a kernel itself
int scratch_address(void** out)
{
    static void* address[64] = {nullptr};
    static std::mutex guard;
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) {
        return fail(HSTU_ERR_RUNTIME, "hipGetDevice failed: %s", hipGetErrorString(err));
    }
    if (dev < 0 || dev >= 64) {
        return fail(HSTU_ERR_RUNTIME, "device index %d is beyond the %d this library keeps scratch addresses for", dev, 64);
    }
    std::lock_guard<std::mutex> lock(guard);
    if (address[dev] == nullptr) {
        void* ptr = nullptr;
        err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (err != hipSuccess || ptr == nullptr) {
            return fail(HSTU_ERR_RUNTIME, "cannot find the scratch array on device %d: %s", dev, hipGetErrorString(err));
        }
        address[dev] = ptr;
    }
    *out = address[dev];
    return HSTU_OK;
}

}  // namespace

extern "C" {

HSTU_API int hstu_jagged_fwd(const hstu_jagged_fwd_params* p, void* workspace, uint64_t workspace_bytes, void* stream)
{
    return launch_forward(p, nullptr, workspace, workspace_bytes, stream);
}

HSTU_API uint64_t hstu_jagged_fwd_noalloc_max_workspace(void) { return kScratchBytes; }

HSTU_API int hstu_jagged_fwd_noalloc(const hstu_jagged_fwd_params* p, void* stream)
{
    const int rc = validate(p);
    if (rc != HSTU_OK) {
        return rc;
    }
    const Variant* var = select(p);
    if (var == nullptr) {
        return HSTU_ERR_UNSUPPORTED;
    }
    const uint64_t need = forward_workspace_bytes(var, p);
    if (need > kScratchBytes) {
        return fail(HSTU_ERR_WORKSPACE,
                    "this call asks for %llu bytes of workspace, the built-in scratch of hstu_jagged_fwd_noalloc holds %llu: "
                    "use hstu_jagged_fwd with a workspace of the caller's",
                    (unsigned long long)need, (unsigned long long)kScratchBytes);
    }
    if (p->total_q == 0) {
        return HSTU_OK;
    }
    void* ptr = nullptr;
    const int rc_scratch = scratch_address(&ptr);
    if (rc_scratch != HSTU_OK) {
        return rc_scratch;
    }
    // (the bytes hstu_jagged_fwd would be given for this description, so that both entry points split items alike)
    return launch_forward(p, nullptr, ptr, need, stream);
}

}  // extern "C"
