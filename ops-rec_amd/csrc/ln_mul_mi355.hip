// C ABI of ln_mul (LayerNorm(x) * u): argument checks, choice of the kernel variant, launch.  Host-side counterpart
// of the reference's adapter checks (ascendc/activation/ln_mul/torch_extension/ln_mul_plugin.cpp:30-51) and of its
// host tiling (ascendc/activation/ln_mul/op_host/ln_mul.cpp:28-92), which cuts the rows over the vector cores; here a
// row goes to a group of lanes sized by the row length.
#include "../../include/ops_rec_activation_mi355.h"

#include <hip/hip_runtime.h>

#include "hstu_error.h"
#include "ln_mul_kernel.hip.h"

namespace {

using hstu::LnMulArgs;

struct LnVariant {
    const char* name;
    void (*kernel)(const LnMulArgs);
    int lanes_per_row;
    int max_chunks;  // 16-byte chunks of a row the variant holds in registers; 0: any row, element by element
};

#define LN_VEC(tag, tagname, G, NV) \
    {"ln_mul_" tagname "_g" #G "_v" #NV, hstu::ln_mul_kernel<hstu::tag, G, NV, true>, G, (G) * (NV)}
#define LN_ANY(tag, tagname, G) {"ln_mul_" tagname "_g" #G "_any", hstu::ln_mul_kernel<hstu::tag, G, 1, false>, G, 0}
// By growing capacity (lanes x chunks per lane); a row takes the first variant that holds it.  Measured on MI355X: a
// tight fit with few chunks per lane streams fastest (lanes past the end of a row still issue their loads), and rows
// of up to 64 chunks do better with several rows per wavefront than with one; the two element-wise forms (short
// rows, long rows) come last.
#define LN_TABLE(tag, tagname)                                                                                        \
    {LN_VEC(tag, tagname, 8, 1),   LN_VEC(tag, tagname, 16, 1),  LN_VEC(tag, tagname, 8, 3),   LN_VEC(tag, tagname, 16, 2),  \
     LN_VEC(tag, tagname, 16, 3),  LN_VEC(tag, tagname, 16, 4),  LN_VEC(tag, tagname, 32, 3),  LN_VEC(tag, tagname, 64, 2),  \
     LN_VEC(tag, tagname, 64, 3),  LN_VEC(tag, tagname, 64, 4),  LN_VEC(tag, tagname, 64, 6),  LN_VEC(tag, tagname, 64, 8),  \
     LN_VEC(tag, tagname, 256, 3), LN_VEC(tag, tagname, 256, 4), LN_VEC(tag, tagname, 256, 6), LN_VEC(tag, tagname, 256, 8), \
     LN_VEC(tag, tagname, 256, 12), LN_VEC(tag, tagname, 256, 16), LN_ANY(tag, tagname, 64),   LN_ANY(tag, tagname, 256)}
constexpr int kVecVariants = 18;
const LnVariant kVariants[3][kVecVariants + 2] = {LN_TABLE(ln_bf16_tag, "bf16"), LN_TABLE(ln_f16_tag, "f16"),
                                                  LN_TABLE(ln_f32_tag, "f32")};

int validate(const ln_mul_params* p)
{
    if (p == nullptr) {
        return hstu::set_error(HSTU_ERR_NULLPTR, "params is NULL");
    }
    if (p->struct_size != sizeof(ln_mul_params)) {
        return hstu::set_error(HSTU_ERR_INVALID, "struct_size %u does not match this library (%zu)", p->struct_size,
                               sizeof(ln_mul_params));
    }
    if (p->x == nullptr || p->u == nullptr || p->gamma == nullptr || p->beta == nullptr || p->out == nullptr) {
        return hstu::set_error(HSTU_ERR_NULLPTR, "x, u, gamma, beta and out must all be given");
    }
    if (p->rows < 1 || p->cols < 1) {
        return hstu::set_error(HSTU_ERR_INVALID, "x tensor must be non-empty (got [%lld, %lld])",
                               static_cast<long long>(p->rows), static_cast<long long>(p->cols));
    }
    if (p->dtype != HSTU_DT_FP32 && p->dtype != HSTU_DT_BF16 && p->dtype != HSTU_DT_FP16) {
        return hstu::set_error(HSTU_ERR_INVALID, "dtype %d is not one of fp32, bf16, fp16", p->dtype);
    }
    if (p->affine_dtype != HSTU_DT_FP32 && p->affine_dtype != p->dtype) {
        return hstu::set_error(HSTU_ERR_INVALID, "gamma / beta must be fp32 or of the type of x (got %d for %d)",
                               p->affine_dtype, p->dtype);
    }
    if (!(p->epsilon >= 0.0f)) {
        return hstu::set_error(HSTU_ERR_INVALID, "epsilon must not be negative");
    }
    if (p->rows > (int64_t{1} << 31) - 1) {
        return hstu::set_error(HSTU_ERR_INVALID, "more than 2^31 - 1 rows");
    }
    return HSTU_OK;
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

const LnVariant* select(const ln_mul_params* p)
{
    const LnVariant* table = kVariants[p->dtype == HSTU_DT_BF16 ? 0 : (p->dtype == HSTU_DT_FP16 ? 1 : 2)];
    const int per_chunk = p->dtype == HSTU_DT_FP32 ? 4 : 8;
    const bool vec_ok = p->cols % per_chunk == 0 && aligned16(p->x) && aligned16(p->u) && aligned16(p->out) &&
                        aligned16(p->gamma) && aligned16(p->beta);
    if (vec_ok) {
        const int64_t chunks = p->cols / per_chunk;
        for (int i = 0; i < kVecVariants; ++i) {
            if (chunks <= table[i].max_chunks) {
                return &table[i];
            }
        }
    }
    return &table[p->cols <= 1024 ? kVecVariants : kVecVariants + 1];
}

}  // namespace

extern "C" {

HSTU_API const char* ln_mul_fwd_kernel_name(const ln_mul_params* params)
{
    return validate(params) == HSTU_OK ? select(params)->name : nullptr;
}

HSTU_API int ln_mul_fwd(const ln_mul_params* p, void* stream)
{
    const int rc = validate(p);
    if (rc != HSTU_OK) {
        return rc;
    }
    const LnVariant* v = select(p);
    LnMulArgs a;
    a.x = p->x;
    a.u = p->u;
    a.gamma = p->gamma;
    a.beta = p->beta;
    a.out = p->out;
    a.rows = p->rows;
    a.cols = p->cols;
    a.epsilon = p->epsilon;
    a.affine_f32 = p->affine_dtype == HSTU_DT_FP32 ? 1 : 0;
    const int rows_per_wg = hstu::kLnMulThreads / v->lanes_per_row;
    const int64_t grid = (p->rows + rows_per_wg - 1) / rows_per_wg;
    hipLaunchKernelGGL(v->kernel, dim3(static_cast<unsigned>(grid)), dim3(hstu::kLnMulThreads), 0,
                       static_cast<hipStream_t>(stream), a);
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        return hstu::set_error(HSTU_ERR_RUNTIME, "launch of %s failed: %s", v->name, hipGetErrorString(err));
    }
    return HSTU_OK;
}

}  // extern "C"
