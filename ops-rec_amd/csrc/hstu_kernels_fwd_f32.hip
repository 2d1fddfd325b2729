// forward kernels for fp32 inputs, the forward and backward kernels for the shapes no tuned kernel takes, and the
// paged gather kernel
#include "hstu_bwd_generic_kernel.hip.h"
#include "hstu_fwd_f32_kernel.hip.h"
#include "hstu_fwd_generic_kernel.hip.h"
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
const Variant kGeneric[3] = {HSTU_GENERIC_VARIANT(__bf16, "bf16"), HSTU_GENERIC_VARIANT(_Float16, "f16"),
                             HSTU_GENERIC_VARIANT(float, "f32")};
}  // namespace
const Variant* fwd_variants_generic() { return kGeneric; }

namespace {
#define HSTU_GENERIC_BWD_VARIANT(T, name) \
    {"hstu_bwd_generic_" name, hstu_bwd_generic_dkv_kernel<T>, hstu_bwd_generic_dq_kernel<T>, hstu_bwd_generic_dq_kernel<T>}
const BwdVariant kGenericBwd[3] = {HSTU_GENERIC_BWD_VARIANT(__bf16, "bf16"), HSTU_GENERIC_BWD_VARIANT(_Float16, "f16"),
                                   HSTU_GENERIC_BWD_VARIANT(float, "f32")};
}  // namespace
const BwdVariant* bwd_variants_generic() { return kGenericBwd; }

void launch_paged_gather(const PagedGatherArgs& a, unsigned grid, hipStream_t stream)
{
    hipLaunchKernelGGL(hstu_paged_gather_kernel, dim3(grid), dim3(kGatherThreads), 0, stream, a);
}
}  // namespace hstu
