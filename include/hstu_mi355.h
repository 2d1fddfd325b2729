/*
 * hstu_mi355.h -- C ABI of the MI355X (gfx950) HSTU jagged attention forward library.
 *
 * This is the native boundary underneath the torch adapter.  It replaces the two-phase
 * C API the reference's adapter binds for this path:
 *
 *   aclnnHstuJaggedForwardGetWorkspaceSize(q, k, v, mask, attnBias, seqOffsetQ, seqOffsetK,
 *        numContext, numTarget, maskType, maxSeqLenQ, maxSeqLenK, siluScale, targetGroupSize,
 *        alpha, deterministic, attnOutput, &workspaceSize, &executor)
 *   aclnnHstuJaggedForward(workspace, workspaceSize, executor, stream)
 *
 *   documented at  ascendc/attention/hstu_v1/hstu_forward_v1/docs/aclnn_hstu_forward.md:50-62
 *   called from    ascendc/attention/hstu_v1/torch_extension/hstu_jagged_plugin.cpp:63-65
 *   C usage        ascendc/attention/hstu_v1/hstu_forward_v1/examples/aclnn/test_aclnn_hstu_forward_jagged.cpp:97-110
 *
 * Conventions kept from that API: C linkage, status-int returns (0 = success), caller owns
 * every buffer including the workspace, optional inputs are NULL, the launch is enqueued on the
 * caller's stream and returns before completion.  Differences: tensors are described by one
 * plain struct of device pointers and sizes instead of opaque handles, and there is no executor
 * object (the library keeps no per-call state, on the host or on the device).
 *
 * The library never allocates or frees device memory and never synchronises the device.
 */
#ifndef HSTU_MI355_H
#define HSTU_MI355_H

#include <stdint.h>

#if defined(__GNUC__)
#define HSTU_API __attribute__((visibility("default")))
#else
#define HSTU_API
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* status codes; the two 1610xx values are the ones the reference documents
 * (aclnn_hstu_forward.md:109-114: 161001 null pointer, 161002 invalid parameter) */
#define HSTU_OK 0
#define HSTU_ERR_NULLPTR 161001
#define HSTU_ERR_INVALID 161002
#define HSTU_ERR_UNSUPPORTED 161003 /* valid for the reference, not (yet) built here */
#define HSTU_ERR_WORKSPACE 161004   /* workspace missing or too small */
#define HSTU_ERR_RUNTIME 561000     /* the HIP runtime reported an error at launch */

/* element types of q/k/v (and of mask / attn_bias, which follow q) */
#define HSTU_DT_BF16 0
#define HSTU_DT_FP16 1
#define HSTU_DT_FP32 2
#define HSTU_DT_FP8_E4M3 3 /* OCP e4m3fn */

/* element type of seq_offset_q / seq_offset_k / num_context / num_target */
#define HSTU_IDX_I32 0
#define HSTU_IDX_I64 1

/* mask_type values (ascendc/attention/hstu_v1/torch_extension/hstu_common.h:47-50) */
#define HSTU_MASK_TRIL 0
#define HSTU_MASK_TRIU 1 /* rejected, as in the reference */
#define HSTU_MASK_NONE 2
#define HSTU_MASK_CUSTOM 3

/* limits (hstu_common.h:31-45, op_host/tiling_policy.cpp:68-93) */
#define HSTU_MAX_BATCH 2048
#define HSTU_MAX_SEQ_LEN 20480
#define HSTU_MAX_HEADS 16
#define HSTU_MAX_HEAD_DIM 512

typedef struct hstu_jagged_fwd_params {
    uint32_t struct_size; /* sizeof(hstu_jagged_fwd_params), checked by the library */
    int32_t dtype;        /* HSTU_DT_* of q, k, v, mask, attn_bias */
    int32_t out_dtype;    /* HSTU_DT_* of out: same as dtype; fp8 input -> HSTU_DT_FP16 (reference) or HSTU_DT_BF16 */
    int32_t index_dtype;  /* HSTU_IDX_* */

    const void* q;            /* [total_q, num_heads_q, head_dim_qk], contiguous, device */
    const void* k;            /* [total_k, num_heads_k, head_dim_qk] */
    const void* v;            /* [total_k, num_heads_k, head_dim_v] */
    const void* mask;         /* NULL or [batch, num_heads_q, max_seq_len_q, max_seq_len_k]; read iff mask_type == 3 */
    const void* attn_bias;    /* NULL or [batch, num_heads_q, max_seq_len_q, max_seq_len_k] */
    const void* seq_offset_q; /* [n_offsets], non-decreasing, first element 0, no span longer than max_seq_len_q
                                 (rows before the first offset, and rows of a sequence past max_seq_len_q, belong to
                                 no work item: the kernels neither read nor write them, so `out` keeps whatever the
                                 caller's buffer held there; the reference's adapter hands out zeros) */
    const void* seq_offset_k; /* [n_offsets]; may equal seq_offset_q */
    const void* num_context;  /* NULL (= zeros) or [n_offsets - 1] */
    const void* num_target;   /* NULL (= zeros) or [n_offsets - 1] */
    void* out;                /* [total_q, num_heads_q, head_dim_v]; every row is written (rows past the last
                                 offset are zero-filled), so the caller need not clear it.  A 16-byte aligned
                                 pointer (any torch allocation) lets the rows be written as whole cache lines;
                                 other pointers work, a few percent slower */

    int64_t total_q;
    int64_t total_k;
    int64_t num_heads_q;
    int64_t num_heads_k;
    int64_t head_dim_qk;
    int64_t head_dim_v;
    int64_t n_offsets; /* batch + 1 */

    int64_t mask_type;
    int64_t max_seq_len_q;
    int64_t max_seq_len_k;
    int64_t target_group_size;
    double silu_scale; /* already resolved by the caller (0.0 is treated as 1 / max_seq_len_q here too) */
    double alpha;
    int32_t deterministic; /* accepted for signature parity; results are bitwise reproducible either way */
    int32_t fp8_scaled_p;  /* fp8 inputs only.  1: P = e4m3(silu(X) * silu_scale * M), the reference's rounding point
                              (op_kernel/atlas950/hstu_dense_forward_kernel_patten_bsnd.h:448-459; with the default
                              silu_scale = 1 / max_seq_len most of P then falls below e4m3's range);
                              0: P = e4m3(silu(X) * M), silu_scale applied to the fp32 output */

    /* fp8 inputs (dtype HSTU_DT_FP8_E4M3, OCP e4m3fn; the reference takes them on its 950 target,
     * op_host/atlas950/op_def_arch.h:23-24): S is kept in fp32, P is clamped to +-448 and re-quantised to
     * e4m3 (round to nearest even), P.V accumulates in fp32, the output is fp16 (the reference's choice,
     * torch_extension/hstu_jagged_plugin.cpp:53-54) or bf16.  attn_bias and a custom mask, when given, are e4m3
     * tensors as well (they follow q's type, op_host/hstu_jagged_forward.cpp:65-66) and are used in fp32; such calls
     * run on the fixed schedule or, for long lists, on the per-XCD queues (their items are not split).  Head dims above 256 and a head_dim_qk that is
     * not a multiple of 16 run on the coverage kernel (vector unit, same semantics).  Where
     * silu_scale is applied relative to the rounding of P is chosen by fp8_scaled_p above.
     * Extension with no counterpart in the reference (its fp8 path is unscaled): per-head dequantisation
     * scales, x = x8 * descale[head]; device pointers, NULL = 1.0.  Ignored unless dtype is fp8. */
    const float* q_descale; /* [num_heads_q] */
    const float* k_descale; /* [num_heads_k] */
    const float* v_descale; /* [num_heads_k] */
} hstu_jagged_fwd_params;

/* replaces aclnnHstuJaggedForwardGetWorkspaceSize: validates the description and reports the scratch
 * size (may be 0).  No device work.
 * Scratch is asked for by two kinds of calls.  A work list that may be several times longer than the machine
 * (long, jagged batches) runs on per-XCD work queues and needs 16 KiB for their counters.  A work list that may be
 * shorter than the machine (few, long sequences) cuts the key range of long items into parts that run on different
 * workgroups and adds their fp32 partial outputs, in a fixed order: 16 KiB of counters plus room for one partial
 * output per resident workgroup.  Lists in between run on a fixed schedule and need nothing.  The workspace is 16-byte
 * aligned; its contents are undefined before and after the call (the library clears the counters on the launch
 * stream ahead of its kernel) and it belongs to the call until the launch has completed: launches that overlap
 * on a GPU -- several streams, captured graphs replayed side by side -- are independent of each other as long as
 * each has a workspace (and an output) of its own.  The library keeps no device state between calls.
 * A caller that passes less than asked for, or nothing, gets the same results from the fixed schedule.  Because a
 * split changes the order of the fp32 sums, the last bit of an output element may then depend on what else is in
 * the batch; HSTU_MI355_SPLIT=0 in the environment turns the split off. */
HSTU_API int hstu_jagged_fwd_workspace_size(const hstu_jagged_fwd_params* params, uint64_t* workspace_bytes);

/* replaces aclnnHstuJaggedForward: enqueues the forward on `stream` (a hipStream_t passed as void*;
 * NULL = the default stream) and returns without waiting for it. */
HSTU_API int hstu_jagged_fwd(const hstu_jagged_fwd_params* params, void* workspace, uint64_t workspace_bytes, void* stream);

/* hstu_jagged_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid it).  No counterpart in the reference.  Same results as hstu_jagged_fwd called with
 * the workspace hstu_jagged_fwd_workspace_size reports, but the workspace is a device array of the library itself
 * (32 MiB + 16 KiB per GPU, held from the first use of the library on that GPU until the process ends): the call
 * takes inputs and outputs only and calls no hipMalloc, hipFree or other allocating routine.  A description whose
 * workspace request exceeds that array (hstu_jagged_fwd_noalloc_max_workspace) is refused with HSTU_ERR_WORKSPACE
 * and nothing is launched.  All calls on one GPU share the one array: two calls that overlap there (different
 * streams, replays of two graphs side by side) race on it and are the caller's to serialise; calls that follow each
 * other on a stream are safe, whatever their sizes (the counters are cleared ahead of every launch). */
HSTU_API int hstu_jagged_fwd_noalloc(const hstu_jagged_fwd_params* params, void* stream);
HSTU_API uint64_t hstu_jagged_fwd_noalloc_max_workspace(void);

/* ---- backward ------------------------------------------------------------------------------------------
 * Replaces the two-phase pair the reference's adapter binds for the backward of this path:
 *
 *   aclnnHstuJaggedBackwardGetWorkspaceSize(grad, q, k, v, mask, attnBias, seqOffsetQ, seqOffsetK, numContext,
 *        numTarget, layout, maskType, maxSeqLenQ, maxSeqLenK, siluScale, targetGroupSize, alpha,
 *        qGrad, kGrad, vGrad, attnBiasGrad, &workspaceSize, &executor)
 *   aclnnHstuJaggedBackward(workspace, workspaceSize, executor, stream)
 *
 *   documented at  ascendc/attention/hstu_v1/hstu_backward_v1/docs/aclnn_hstu_jagged_backward.md:24-56
 *   C usage        ascendc/attention/hstu_v1/hstu_backward_v1/examples/aclnn/test_aclnn_hstu_backward_v1_jagged.cpp:174-186
 *
 * `fwd` describes q, k, v, mask, attn_bias, the offsets and the scalars exactly as for the forward (fwd.out is
 * not used and may be NULL).  bf16 / fp16 with head dims up to 256 and a q/k head dim that is a multiple of 8 run
 * on the tuned kernels, and so do head dims in (256, 512] that are multiples of 16 (as two windows per head; this
 * needs the workspace, see below); fp32 with head dims up to 128 and a q/k head dim that is a multiple of 8 runs on
 * kernels built on the fp32 matrix instruction; every other input the forward takes runs on generic fp32-arithmetic
 * kernels (correct, slow).  fp8 inputs return HSTU_ERR_UNSUPPORTED.
 * grad_q / grad_k / grad_v: every row is written (rows past the last offset are zero-filled), so the caller
 * need not clear them.  grad_attn_bias (optional; requires attn_bias): written in full as well -- zeros outside
 * the part of a sequence's [S_q, S_k] corner that its query tiles sweep -- so the caller need not clear it either
 * (the first kernel of the call clears it beside its work).
 * Workspace (optional): the tuned kernels recompute nothing, or less, when the query-tile kernel's dS (and P) have
 * somewhere to stay until the kernels that produce grad_k (and grad_v) read them back: dS in grad_attn_bias (which
 * is dS) when that is asked for, otherwise in a workspace of [batch, num_heads_q, max_seq_len_q, max_seq_len_k]
 * elements of the input type; dS and P together in a workspace of one 128-byte line per head, query row of the batch
 * and 32-key block (only the blocks at or below the diagonal for a causal mask over equal query and key offsets
 * without context rows; otherwise ceil(max_seq_len_k / 32) | 1 lines per row).  hstu_jagged_bwd_workspace_size asks for the workspace of the order it estimates to be the
 * fastest (at most 2 GiB -- 16 GiB at head dims above 128, where it saves a good part of the call -- or HSTU_MI355_BWD_WORKSPACE_MB in the environment; with an attn_bias, a custom mask or an
 * attn_bias gradient, or for the [batch, ...] plane of dS alone, max_seq_len_k must be a multiple of 4 -- rows of such
 * tensors are read and written in pieces of 8 keys, one 16-byte access when max_seq_len_k is a multiple of 8, two
 * 8-byte ones otherwise -- while the workspace for dS and P together has its own layout; fp32
 * inputs with head dims up to 128: dS and P in fp32 whenever that fits).  Head dims above 256 need, beside that line
 * per row and block, 256 bytes per head, query row and block for the scores of the first window.  Without the workspace,
 * or with less than was asked for, the call still works: the kernels that produce grad_k then recompute dS (head dims
 * above 256: the generic kernels run).  The workspace needs no clearing and holds nothing afterwards.  Batches of
 * sequences of at most 32 rows and keys (bf16 / fp16, no attn_bias, no custom mask, head dims up to 256 in multiples
 * of 8, 16-byte aligned tensors) run in one launch and ask for no workspace, and so do batches of sequences of at most
 * 64 query rows against keys of any length at head dims up to 128 with num_heads_k == num_heads_q. */
typedef struct hstu_jagged_bwd_params {
    uint32_t struct_size; /* sizeof(hstu_jagged_bwd_params) */
    uint32_t reserved0;
    hstu_jagged_fwd_params fwd;
    const void* grad;     /* [total_q, num_heads_q, head_dim_v], dtype of q */
    void* grad_q;         /* [total_q, num_heads_q, head_dim_qk] */
    void* grad_k;         /* [total_k, num_heads_k, head_dim_qk] */
    void* grad_v;         /* [total_k, num_heads_k, head_dim_v] */
    void* grad_attn_bias; /* NULL or [batch, num_heads_q, max_seq_len_q, max_seq_len_k] */
} hstu_jagged_bwd_params;

HSTU_API int hstu_jagged_bwd_workspace_size(const hstu_jagged_bwd_params* params, uint64_t* workspace_bytes);
HSTU_API int hstu_jagged_bwd(const hstu_jagged_bwd_params* params, void* workspace, uint64_t workspace_bytes, void* stream);

/* ---- paged K/V ---------------------------------------------------------------------------------------
 * Replaces the pair the reference's adapter binds for hstu_paged (inference with a paged KV cache):
 *
 *   aclnnHstuPagedForward[GetWorkspaceSize](q, k, v, mask, attnBias, seqOffset, seqOffsetK, seqOffsetT, kvCache,
 *        pageOffsets, pageIds, lastPageLen, numContext, numTarget, maskType, maxSeqLen, maxSeqLenK, siluScale,
 *        targetGroupSize, alpha, deterministic, attnOutput)
 *   called from  ascendc/attention/hstu_v1/torch_extension/hstu_paged_plugin.cpp:66-69
 *
 * The keys / values of sequence b are its cached rows -- the pages page_ids[page_offsets[b] .. page_offsets[b+1])
 * of kv_cache [num_pages, 2 (K, V), page_size, num_heads_k, head_dim], in order -- followed by the rows of its
 * num_target[b] new target tokens, which are the LAST num_target[b] rows of its segment [seq_offset_q[b],
 * seq_offset_q[b+1]) of the k / v inputs (the other rows of k / v are not read).  fwd.seq_offset_k gives the
 * resulting key ranges (cached + targets per sequence) and fwd.total_k an upper bound on their end
 * (page_ids count x page_size + total_q is always enough); fwd.k / fwd.v MUST hold total_q rows each (the new rows
 * are addressed by query row index, bounded by total_q only; the torch adapter checks the row counts);
 * fwd.num_context is ignored (zeros, as in the reference adapter); everything else as in the forward.
 * Implementation: for bf16 / fp16 with head dims up to 128 the forward kernel reads the pages itself (a page
 * look-up per 32-key sub-tile, page_size being a multiple of 32); the workspace then holds 16 KiB of work counters
 * (required: HSTU_ERR_WORKSPACE without them) and the optional room for splitting long key ranges over workgroups,
 * as in hstu_jagged_fwd.  Otherwise (fp32, larger head dims) the library
 * first gathers the rows into the workspace (one copy kernel: 2 x total_k rows, required) and runs the jagged
 * forward on them.  last_page_len and seq_offset_t are taken for signature parity and never read: the number of
 * cached rows of a sequence is its key count minus its targets, so page metadata that disagrees with
 * fwd.seq_offset_k / fwd.num_target is the caller's to keep consistent. */
typedef struct hstu_paged_fwd_params {
    uint32_t struct_size; /* sizeof(hstu_paged_fwd_params) */
    uint32_t reserved0;
    hstu_jagged_fwd_params fwd;
    const void* kv_cache;      /* dtype of q */
    const void* page_offsets;  /* [n_offsets], index dtype */
    const void* page_ids;      /* [n_page_ids] */
    const void* last_page_len; /* [n_offsets - 1]; may be NULL */
    const void* seq_offset_t;  /* [n_offsets]; may be NULL */
    int64_t num_pages;
    int64_t page_size;
    int64_t n_page_ids;
} hstu_paged_fwd_params;

HSTU_API int hstu_paged_fwd_workspace_size(const hstu_paged_fwd_params* params, uint64_t* workspace_bytes);
HSTU_API int hstu_paged_fwd(const hstu_paged_fwd_params* params, void* workspace, uint64_t workspace_bytes, void* stream);

/* replaces aclGetRecentErrMsg (ascendc/common/torch_plugin/pytorch_npu_helper.hpp:649,662):
 * text of the calling thread's most recent failure; never NULL. */
HSTU_API const char* hstu_last_error(void);

/* The library's process-wide switches (HSTU_MI355_SPLIT, HSTU_MI355_SHORT, HSTU_MI355_GENERIC_BACKWARD,
 * HSTU_MI355_BWD_HANDOFF, HSTU_MI355_BWD_WORKSPACE_MB, HSTU_MI355_BWD_PAIR_MAJOR) are read from the environment once, at the first call that
 * looks at one; this reads them again.  No counterpart in the reference: it is for a test or a tool that changes the
 * environment after the library has been used.  Not safe against launches running at the same time in other threads. */
HSTU_API void hstu_reload_switches(void);

/* library version, (major << 16) | minor */
HSTU_API int hstu_version(void);

/* name of the kernel variant hstu_jagged_fwd would launch for `params` (for profiles and logs),
 * or NULL after an error.  The string is static. */
HSTU_API const char* hstu_jagged_fwd_kernel_name(const hstu_jagged_fwd_params* params);

#ifdef __cplusplus
}
#endif
#endif /* HSTU_MI355_H */
