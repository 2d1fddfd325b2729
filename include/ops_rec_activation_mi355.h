/*
 * C ABI of the MI355X (gfx950) build of the operators around HSTU attention in an HSTU layer.  Same library, status
 * codes, dtype codes and error text (hstu_last_error) as hstu_mi355.h.
 *
 * Two operators: ln_mul (consumes the attention output) and in_linear_silu (produces U, V, Q, K in front of it).
 *
 * ln_mul: out = LayerNorm(x) * u over the rows of a [rows, cols] matrix, with
 *   LayerNorm(x) = (x - mean) * rstd * gamma + beta,  rstd = 1 / sqrt(var + epsilon),  var = mean((x - mean)^2).
 *
 * Replaces the two-phase pair aclnnLnMulGetWorkspaceSize / aclnnLnMul
 * (ascendc/activation/ln_mul/docs/aclnn_ln_mul.md:26-41), which the reference's torch adapter calls through
 * EXEC_NPU_CMD (ascendc/activation/ln_mul/torch_extension/ln_mul_plugin.cpp:49).  The aclTensor handles become plain
 * device pointers plus the two extents; the op needs no workspace, so one call does both phases.
 *
 * Beyond the reference (fp32 only, ascendc/activation/ln_mul/op_host/ln_mul.cpp:111-135): x / u / out may be bf16
 * or fp16 (the types the attention kernels write), with gamma / beta in fp32 or in that type; arithmetic is fp32.
 */
#ifndef OPS_REC_ACTIVATION_MI355_H
#define OPS_REC_ACTIVATION_MI355_H

#include "hstu_mi355.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ln_mul_params {
    uint32_t struct_size; /* sizeof(ln_mul_params), checked */
    uint32_t reserved0;
    const void* x;     /* [rows, cols], contiguous */
    const void* u;     /* [rows, cols], contiguous */
    const void* gamma; /* [cols] */
    const void* beta;  /* [cols] */
    void* out;         /* [rows, cols]; every element is written */
    int64_t rows;
    int64_t cols;
    int32_t dtype;        /* of x, u, out: HSTU_DT_FP32 (the reference's), HSTU_DT_BF16, HSTU_DT_FP16 */
    int32_t affine_dtype; /* of gamma, beta: HSTU_DT_FP32 or equal to dtype */
    float epsilon;        /* the reference fixes 1e-5 (ascendc/activation/ln_mul/op_host/ln_mul.cpp:75) */
    uint32_t reserved1;
} ln_mul_params;

/* Launches the kernel on `stream` (a hipStream_t; NULL = the default stream) and returns without waiting.
 * HSTU_OK, or HSTU_ERR_NULLPTR / HSTU_ERR_INVALID (nothing launched) / HSTU_ERR_RUNTIME. */
HSTU_API int ln_mul_fwd(const ln_mul_params* params, void* stream);

/* name of the kernel variant ln_mul_fwd would launch (for profiles and logs), or NULL after an error */
HSTU_API const char* ln_mul_fwd_kernel_name(const ln_mul_params* params);

/*
 * in_linear_silu forward: mixed = x @ weight^T + bias; linear_output = mixed; (user, value, query, key) =
 * split(silu(mixed), split, last dim).  linear_output is mixed rounded to the type of x, and SiLU is taken of that
 * rounded value, as the reference's kernel does.
 *
 * Replaces the two-phase pair aclnnInLinearSiluGetWorkspaceSize / aclnnInLinearSilu
 * (ascendc/activation/in_linear_silu/in_linear_silu_forward/docs/aclnn_in_linear_silu.md), which the reference's torch
 * adapter calls through EXEC_NPU_CMD (ascendc/activation/in_linear_silu/torch_extension/in_linear_silu_plugin.cpp:85-86).
 * Limits as in that adapter (in_linear_silu_plugin.cpp:36-66): k in [16, 8192] and n in [64, 32768], multiples of 16;
 * every split in [16, 8192], a multiple of 16, the four adding up to n; n a multiple of 4 k.
 */
typedef struct in_linear_silu_params {
    uint32_t struct_size; /* sizeof(in_linear_silu_params), checked */
    uint32_t reserved0;
    const void* x;       /* [m, k], bf16 or fp16, contiguous, 16-byte aligned */
    const void* weight;  /* [n, k], type of x */
    const float* bias;   /* [n] fp32, or NULL for no bias */
    void* user;          /* [m, split[0]], type of x */
    void* value;         /* [m, split[1]] */
    void* query;         /* [m, split[2]] */
    void* key;           /* [m, split[3]] */
    void* linear_output; /* [m, n] */
    int64_t m;
    int64_t n;
    int64_t k;
    int64_t split[4];
    int32_t dtype; /* HSTU_DT_BF16 or HSTU_DT_FP16 */
    uint32_t reserved1;
} in_linear_silu_params;

/* Launches the kernel on `stream` and returns without waiting.  HSTU_OK, or HSTU_ERR_NULLPTR / HSTU_ERR_INVALID
 * (nothing launched) / HSTU_ERR_RUNTIME. */
HSTU_API int in_linear_silu_fwd(const in_linear_silu_params* params, void* stream);

/* name of the kernel variant in_linear_silu_fwd would launch, or NULL after an error */
HSTU_API const char* in_linear_silu_fwd_kernel_name(const in_linear_silu_params* params);

/*
 * The element-wise stage of in_linear_silu's backward (the reference does the whole backward in one call,
 * aclnnInLinearSiluBackward, ascendc/activation/in_linear_silu/in_linear_silu_backward/docs/aclnn_in_linear_silu_backward.md;
 * its adapter: torch_extension/in_linear_silu_backward_plugin.cpp:112-153):
 *   d_mixed = cat(user_grad, value_grad, query_grad, key_grad) * silu'(linear_output),  bias_grad = column sums.
 * The two products that follow (d x = d_mixed @ weight, d weight = d_mixed^T @ x) are plain matrix products and are left
 * to the caller's BLAS.
 */
typedef struct in_linear_silu_bwd_params {
    uint32_t struct_size; /* sizeof(in_linear_silu_bwd_params), checked */
    uint32_t reserved0;
    const void* linear_output; /* [m, n], bf16 or fp16: the forward's fifth output */
    const void* user_grad;     /* [m, split[0]], same type */
    const void* value_grad;    /* [m, split[1]] */
    const void* query_grad;    /* [m, split[2]] */
    const void* key_grad;      /* [m, split[3]] */
    void* d_mixed;             /* [m, n], same type; every element is written */
    float* bias_grad;          /* [n] fp32, or NULL when there is no bias */
    int64_t m;
    int64_t n;
    int64_t split[4];
    int32_t dtype; /* HSTU_DT_BF16 or HSTU_DT_FP16 */
    uint32_t reserved1;
} in_linear_silu_bwd_params;

/* bytes of device scratch in_linear_silu_bwd_dmixed needs (partial column sums: ceil(m / 64) * n floats; 0 when
 * bias_grad is NULL) */
HSTU_API int in_linear_silu_bwd_dmixed_workspace_size(const in_linear_silu_bwd_params* params, uint64_t* workspace_bytes);

/* Launches on `stream` and returns without waiting.  HSTU_OK, or HSTU_ERR_NULLPTR / HSTU_ERR_INVALID /
 * HSTU_ERR_WORKSPACE (nothing launched) / HSTU_ERR_RUNTIME. */
HSTU_API int in_linear_silu_bwd_dmixed(const in_linear_silu_bwd_params* params, void* workspace, uint64_t workspace_bytes,
                                       void* stream);

#ifdef __cplusplus
}
#endif
#endif
