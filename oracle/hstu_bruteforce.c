/*
 * Scalar CPU restatement of HSTU jagged attention forward.  TEST INFRASTRUCTURE ONLY:
 * it checks the torch oracle (hstu_oracle.py) and the HIP operator, it is never the
 * thing shipped or measured as the product.
 *
 * Plain triple loop, double accumulation, libm exp().  Written independently of the
 * torch oracle on purpose (different loop order, different mask statement) so that a
 * dropped term, a wrong index or a transposed operand in either one shows up as a
 * disagreement.
 *
 * Semantics follow the reference's goldens:
 *   ascendc/attention/hstu_v1/hstu_forward_v1/test/pytest/common.py:189-252
 *       (per-sequence loop, bias slice [b, :, :S_q, :S_k], delta diagonal S_k - S_q)
 *   ascendc/attention/hstu_v2/test/pytest/backend/pytorch_native_backend.py:69-76
 *       (x = alpha * (qk + bias); p = silu(x) * scale; p *= mask)
 *   ascendc/attention/hstu_v1/hstu_forward_v1/op_kernel/atlas950/hstu_dense_causal_mask.h:186-260
 *       (context / causal / target regions of mask_type 0)
 *   ascendc/attention/hstu_v1/hstu_forward_v1/op_kernel/atlas950/hstu_common_const.h:124-147
 *       (effective batch = index of the first offset equal to the last one)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static int visible(int64_t i, int64_t j, int64_t s_q, int64_t s_k, int64_t ctx, int64_t tgt, int64_t group)
{
    int64_t hist_k = s_k - tgt; /* keys before the target block */
    int64_t ti = i - (s_q - tgt); /* row index inside the target block (may be < 0) */
    int64_t tj = j - hist_k;      /* column index inside the target block */
    if (tgt > 0 && group > 0 && ti >= 0 && tj >= 0) {
        return tj <= ti && (ti / group) == (tj / group);
    }
    if (ctx > 0 && i < ctx && j < hist_k) {
        return 1;
    }
    return j - (s_k - s_q) <= i;
}

/* returns 0 on success, non-zero on bad arguments */
int hstu_bruteforce_forward(const float* q, const float* k, const float* v, const float* mask, const float* bias,
                            const int64_t* offs_q, const int64_t* offs_k, const int64_t* num_context,
                            const int64_t* num_target, int64_t n_offsets, int64_t n_q, int64_t n_k, int64_t d_qk,
                            int64_t d_v, int64_t max_q, int64_t max_k, int64_t mask_type, double silu_scale,
                            int64_t target_group_size, double alpha, float* out)
{
    if (n_offsets < 2 || n_k <= 0 || n_q % n_k != 0) {
        return 1;
    }
    if (mask_type == 3 && mask == NULL) {
        return 2;
    }
    if (mask_type != 0 && mask_type != 2 && mask_type != 3) {
        return 3;
    }
    double scale = (silu_scale == 0.0) ? 1.0 / (double)max_q : silu_scale;
    int64_t ratio = n_q / n_k;
    int64_t last = offs_q[n_offsets - 1];
    int64_t batch = n_offsets - 1;
    for (int64_t b = 0; b < n_offsets; ++b) {
        if (offs_q[b] == last) {
            batch = b;
            break;
        }
    }
    memset(out, 0, sizeof(float) * (size_t)(last * n_q * d_v));
    double* acc = (double*)malloc(sizeof(double) * (size_t)d_v);
    if (!acc) {
        return 4;
    }
    for (int64_t b = 0; b < batch; ++b) {
        int64_t q0 = offs_q[b], s_q = offs_q[b + 1] - q0;
        int64_t k0 = offs_k[b], s_k = offs_k[b + 1] - k0;
        int64_t ctx = num_context ? num_context[b] : 0;
        int64_t tgt = num_target ? num_target[b] : 0;
        for (int64_t h = 0; h < n_q; ++h) {
            int64_t hk = h / ratio;
            for (int64_t i = 0; i < s_q; ++i) {
                const float* qrow = q + ((q0 + i) * n_q + h) * d_qk;
                for (int64_t e = 0; e < d_v; ++e) {
                    acc[e] = 0.0;
                }
                for (int64_t j = 0; j < s_k; ++j) {
                    double w = 1.0;
                    if (mask_type == 0) {
                        if (!visible(i, j, s_q, s_k, ctx, tgt, target_group_size)) {
                            continue;
                        }
                    } else if (mask_type == 3) {
                        w = (double)mask[((b * n_q + h) * max_q + i) * max_k + j];
                    }
                    const float* krow = k + ((k0 + j) * n_k + hk) * d_qk;
                    double s = 0.0;
                    for (int64_t e = 0; e < d_qk; ++e) {
                        s += (double)qrow[e] * (double)krow[e];
                    }
                    if (bias) {
                        s += (double)bias[((b * n_q + h) * max_q + i) * max_k + j];
                    }
                    double x = alpha * s;
                    double p = x / (1.0 + exp(-x)) * scale * w;
                    const float* vrow = v + ((k0 + j) * n_k + hk) * d_v;
                    for (int64_t e = 0; e < d_v; ++e) {
                        acc[e] += p * (double)vrow[e];
                    }
                }
                float* orow = out + ((q0 + i) * n_q + h) * d_v;
                for (int64_t e = 0; e < d_v; ++e) {
                    orow[e] = (float)acc[e];
                }
            }
        }
    }
    free(acc);
    return 0;
}

/* the mask predicate alone, for cross-checking the closed form: fills m[s_q * s_k] with 0/1 */
void hstu_bruteforce_mask(int64_t s_q, int64_t s_k, int64_t ctx, int64_t tgt, int64_t group, float* m)
{
    for (int64_t i = 0; i < s_q; ++i) {
        for (int64_t j = 0; j < s_k; ++j) {
            m[i * s_k + j] = visible(i, j, s_q, s_k, ctx, tgt, group) ? 1.0f : 0.0f;
        }
    }
}
