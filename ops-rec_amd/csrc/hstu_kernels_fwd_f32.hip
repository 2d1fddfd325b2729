// forward kernels for fp32 inputs, for 16-bit inputs with head dims in (256, 512], the forward and backward kernels
// for the shapes no other kernel takes, and the paged gather kernel
#include "hstu_bwd_f32_kernel.hip.h"
#include "hstu_bwd_generic_kernel.hip.h"
#include "hstu_fwd_f32_kernel.hip.h"
#include "hstu_fwd_generic_kernel.hip.h"
#include "hstu_fwd_wide_kernel.hip.h"
#include "hstu_paged_gather.hip.h"
#include "hstu_variants.h"

#define HSTU_F32_VARIANT(D, RAB, MASK)                                                                              \
    {"hstu_fwd_f32_d" #D "_rab" #RAB "_mask" #MASK, nullptr, nullptr, hstu::hstu_fwd_f32_kernel<D, RAB, MASK>, nullptr, \
     nullptr, nullptr, D, 256, 0}
#define HSTU_F32_DIMS(RAB, MASK) \
    {HSTU_F32_VARIANT(32, RAB, MASK), HSTU_F32_VARIANT(64, RAB, MASK), HSTU_F32_VARIANT(128, RAB, MASK), \
     HSTU_F32_VARIANT(256, RAB, MASK)}

namespace hstu {
namespace {
const Variant kTable[2][2][4] = {{HSTU_F32_DIMS(false, false), HSTU_F32_DIMS(false, true)},
                                 {HSTU_F32_DIMS(true, false), HSTU_F32_DIMS(true, true)}};
}
const Variant (*fwd_variants_f32())[2][4] { return kTable; }

namespace {
#define HSTU_GENERIC_VARIANT(T, name) \
    {"hstu_fwd_generic_" name, nullptr, nullptr, hstu_fwd_generic_kernel<T>, nullptr, nullptr, nullptr, kGenericMaxDim, 256, 0}
#define HSTU_GENERIC_F8_VARIANT(OutT, name)                                                                           \
    {"hstu_fwd_generic_f8e4m3_" name, nullptr, nullptr, hstu_fwd_generic_kernel<f8e4m3_elem, OutT>, nullptr, nullptr, nullptr, \
     kGenericMaxDim, 256, 0}
// [bf16, fp16, fp32, fp8-e4m3 with fp16 output, fp8-e4m3 with bf16 output]
const Variant kGeneric[5] = {HSTU_GENERIC_VARIANT(__bf16, "bf16"), HSTU_GENERIC_VARIANT(_Float16, "f16"),
                             HSTU_GENERIC_VARIANT(float, "f32"), HSTU_GENERIC_F8_VARIANT(_Float16, "f16"),
                             HSTU_GENERIC_F8_VARIANT(__bf16, "bf16")};
}  // namespace
const Variant* fwd_variants_generic() { return kGeneric; }

namespace {
#define HSTU_WIDE_VARIANT(tag, name, RAB, MASK)                                                                          \
    {"hstu_fwd_wide_" name "_rab" #RAB "_mask" #MASK, nullptr, nullptr, hstu_fwd_wide_kernel<tag, RAB, MASK>, nullptr, nullptr, \
     nullptr, kWideDim, 256, 0}
#define HSTU_WIDE_TYPE(tag, name)                                                                       \
    {{HSTU_WIDE_VARIANT(tag, name, 0, 0), HSTU_WIDE_VARIANT(tag, name, 0, 1)}, \
     {HSTU_WIDE_VARIANT(tag, name, 1, 0), HSTU_WIDE_VARIANT(tag, name, 1, 1)}}
const Variant kWide[2][2][2] = {HSTU_WIDE_TYPE(bf16_tag, "bf16"), HSTU_WIDE_TYPE(f16_tag, "f16")};
}  // namespace
const Variant (*fwd_variants_wide())[2][2] { return kWide; }

namespace {
#define HSTU_GENERIC_BWD_VARIANT(T, name, M)                                                                          \
    {"hstu_bwd_generic_" name "_d" #M, hstu_bwd_generic_dkv_kernel<T, M>, hstu_bwd_generic_dq_kernel<T, M>, \
     hstu_bwd_generic_dq_kernel<T, M>}
#define HSTU_GENERIC_BWD_TYPE(T, name) \
    {HSTU_GENERIC_BWD_VARIANT(T, name, 128), HSTU_GENERIC_BWD_VARIANT(T, name, 256), HSTU_GENERIC_BWD_VARIANT(T, name, 512)}
const BwdVariant kGenericBwd[3][3] = {HSTU_GENERIC_BWD_TYPE(__bf16, "bf16"), HSTU_GENERIC_BWD_TYPE(_Float16, "f16"),
                                      HSTU_GENERIC_BWD_TYPE(float, "f32")};
}  // namespace
const BwdVariant (*bwd_variants_generic())[3] { return kGenericBwd; }

namespace {
#define HSTU_F32_BWD_VARIANT(D, RAB, MASK)                                                                    \
    {"hstu_bwd_f32_d" #D "_rab" #RAB "_mask" #MASK, hstu_bwd_f32_dkv_kernel<D, RAB, MASK>, hstu_bwd_f32_dq_kernel<D, RAB, MASK>, \
     hstu_bwd_f32_dq_kernel<D, RAB, MASK>, nullptr, nullptr, hstu_bwd_f32_dq_kernel<D, RAB, MASK, true>,                  \
     hstu_bwd_f32_dkv_kernel<D, false, false, true>, hstu_bwd_f32_dkv_kernel<D, false, false, true>}
#define HSTU_F32_BWD_DIMS(RAB, MASK) \
    {HSTU_F32_BWD_VARIANT(32, RAB, MASK), HSTU_F32_BWD_VARIANT(64, RAB, MASK), HSTU_F32_BWD_VARIANT(128, RAB, MASK)}
const BwdVariant kF32Bwd[2][2][3] = {{HSTU_F32_BWD_DIMS(0, 0), HSTU_F32_BWD_DIMS(0, 1)},
                                     {HSTU_F32_BWD_DIMS(1, 0), HSTU_F32_BWD_DIMS(1, 1)}};
}  // namespace
const BwdVariant (*bwd_variants_f32())[2][3] { return kF32Bwd; }

void launch_paged_gather(const PagedGatherArgs& a, unsigned grid, hipStream_t stream)
{
    hipLaunchKernelGGL(hstu_paged_gather_kernel, dim3(grid), dim3(kGatherThreads), 0, stream, a);
}
}  // namespace hstu
