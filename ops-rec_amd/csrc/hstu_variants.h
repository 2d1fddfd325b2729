// Tables of kernel variants.  The kernels are instantiated in several translation units (one per input type and
// direction, so that they compile side by side); each unit hands out its table through one of the functions below.
#pragma once
#include <hip/hip_runtime.h>

#include "hstu_args.h"

namespace hstu {

// kernel variants with the per-XCD work queues and with split items exist for the head-dim slots 64 and 128, the one
// with paged keys for 64, 128 and 256 (nullptr elsewhere)
struct Variant {
    const char* name;
    const char* name_queues;
    const char* name_split;
    void (*kernel)(const FwdArgs);
    void (*kernel_queues)(const FwdArgs);  // the same with per-XCD work queues, for long lists; may be nullptr
    void (*kernel_split)(const FwdArgs);   // the same with long items split over workgroups, for short lists
    void (*kernel_paged)(const FwdArgs);   // split variant that reads K / V through a page table; may be nullptr
    int d_pad;
    int threads;
    int persistent_wgs_per_cu;  // > 0: persistent kernel, this many workgroups per CU; 0: one workgroup per tile
};

// the forward kernel for short work lists (hstu_fwd_short_kernel.hip.h): one workgroup of `threads` per
// (query tile, sequence, head) slot, no list, no workspace
struct ShortVariant {
    const char* name;
    void (*kernel)(const FwdArgs);
};

// the whole backward in one launch: for batches of tiny sequences (hstu_bwd_tiny_kernel.hip.h), for sequences of few query
// rows (hstu_bwd_few_rows_kernel.hip.h)
struct BwdTinyVariant {
    const char* name;
    void (*kernel)(const BwdArgs);
};

// the query-tile backward kernel for short rows (hstu_bwd_dq_short_kernel.hip.h): 16-bit inputs, head-dim slot 128,
// no bias, no custom mask; one workgroup of `threads` per (64-row tile, sequence, head) slot
struct DqShortVariant {
    void (*dq)(const BwdArgs);       // dQ only
    void (*dq_ds)(const BwdArgs);    // storing dS (bias layout) for dK workgroups that read it back
    void (*dq_ds_p)(const BwdArgs);  // storing dS and P for the key-tile workgroups that read them back
};

struct BwdVariant {
    const char* name;
    void (*dkv)(const BwdArgs);
    void (*dq)(const BwdArgs);       // without d rab
    void (*dq_drab)(const BwdArgs);  // storing dS (the attn_bias gradient) as well; nullptr in the generic and fp32 tables
    // the three-launch order dV / dQ storing dS / dK from that dS (nullptr in the generic and fp32 tables)
    void (*dv_only)(const BwdArgs);
    void (*dk_from_ds)(const BwdArgs);
    // the order dQ storing dS and P / dV workgroups that read P beside dK workgroups that read dS
    void (*dq_ds_p)(const BwdArgs);
    void (*dv_dk_from_planes)(const BwdArgs);
    void (*dv_dk_from_planes_drab)(const BwdArgs);  // the dK workgroups also write dS to the attn_bias gradient
    // head dims above 256 as two windows per head on the kernels of the slot 256 (nullptr elsewhere): the query-tile kernel
    // over the first window (S and dP to the fp32 partial plane), over the second (dS and P to the pair plane, dQ of that
    // window), and dQ of the first window from the stored dS
    void (*dq_win_first)(const BwdArgs);
    void (*dq_win_second_ds_p)(const BwdArgs);
    void (*dq_win_from_plane)(const BwdArgs);
};

// forward, 16-bit inputs: [rab: 0, 1][custom mask: 0, 1][dim slot: 32, 64, 128, 256]
const Variant (*fwd_variants_bf16())[2][4];
const Variant (*fwd_variants_f16())[2][4];
// forward, fp8-e4m3 inputs: [output: fp16, bf16][rab][custom mask][dim slot: 64, 128, 256]
const Variant (*fwd_variants_f8())[2][2][3];
// forward, fp32 inputs: [rab][custom mask][dim slot: 32, 64, 128, 256]
const Variant (*fwd_variants_f32())[2][4];
// forward, 16-bit inputs with head dims in (256, 512], q/k head dim a multiple of 8: [bf16, fp16][rab][custom mask]
const Variant (*fwd_variants_wide())[2][2];
// forward for short work lists, 16-bit inputs at the head-dim slot 128 without custom mask: [bf16, fp16, bf16 with
// attn_bias, fp16 with attn_bias]
const ShortVariant* fwd_variants_short();
// forward for batches of sequences of at most 32 or 64 rows and keys (hstu_fwd_tiny_kernel.hip.h; one workgroup of four
// threads per row per (sequence, head)), no bias, no custom mask: [bf16, fp16][head-dim slot 64, 128, 256][32, 64 rows]
const ShortVariant (*fwd_variants_tiny())[3][2];
// forward for small launches of sequences of at most 64 query rows against keys of any length (hstu_fwd_few_rows_kernel.hip.h;
// one workgroup of kFwdFewRowsThreads per (sequence, head)), no bias, no custom mask: [bf16, fp16][head-dim slot 64, 128]
const ShortVariant (*fwd_variants_few_rows())[2];
// forward, any head dims up to 512 (written for coverage, not speed): [bf16, fp16, fp32, fp8-e4m3 -> fp16, fp8-e4m3 -> bf16]
const Variant* fwd_variants_generic();
// backward: [rab][custom mask][dim slot: 64, 128, 256]
const BwdVariant (*bwd_variants_bf16())[2][3];
const BwdVariant (*bwd_variants_f16())[2][3];
// backward, query-tile kernel for short rows: [bf16, fp16]
const DqShortVariant* bwd_variants_dq_short();
// backward for batches of sequences of at most 32 rows and keys (one workgroup of kTinyThreads per (sequence, K/V head)),
// no bias, no custom mask, head dims up to 256 in multiples of 8: [bf16, fp16][head-dim slot 128, 256]
const BwdTinyVariant (*bwd_variants_tiny())[2];
// backward for sequences of at most 64 query rows and any number of keys (one workgroup of kFewRowsThreads per (sequence,
// head)), no bias, no custom mask, head dims up to 128 in multiples of 8, as many K/V heads as query heads:
// [bf16, fp16][head-dim slot 64, 128]
const BwdTinyVariant (*bwd_variants_few_rows())[2];
// backward, fp32 inputs with head dims up to 128 (fp32 MFMA, one workgroup per key tile, the same kernel with and
// without d rab; launched like the generic ones, behind fills of the outputs): [rab][custom mask][dim slot: 32, 64, 128]
const BwdVariant (*bwd_variants_f32())[2][3];
// backward, fp32 inputs and any head dims up to 512 (written for coverage, not speed; one workgroup per key tile,
// the same kernel with and without d rab): [bf16, fp16, fp32][head dims up to 128, 256, 512]
const BwdVariant (*bwd_variants_generic())[3];
// the copy kernel in front of the forward for paged keys that no paged kernel variant covers
void launch_paged_gather(const PagedGatherArgs& a, unsigned grid, hipStream_t stream);

}  // namespace hstu
