// backward kernels for bf16 inputs
#include "hstu_bwd_kernel.hip.h"
#include "hstu_variants.h"

namespace hstu {
namespace {
#define HSTU_BWD_VARIANT(D, RAB, MASK, WIN)                                                       \
    {"hstu_bwd_bf16_d" #D "_rab" #RAB "_mask" #MASK, hstu_bwd_dkv_kernel<bf16_tag, D, RAB, MASK>, \
     hstu_bwd_dq_kernel<bf16_tag, D, RAB, MASK, 0>, hstu_bwd_dq_kernel<bf16_tag, D, RAB, MASK, 1>, \
     hstu_bwd_dkv_kernel<bf16_tag, D, RAB, MASK, 1>, hstu_bwd_dkv_kernel<bf16_tag, D, false, false, 2>, \
     hstu_bwd_dq_kernel<bf16_tag, D, RAB, MASK, 2>, hstu_bwd_dkv_kernel<bf16_tag, D, false, false, 4>, \
     hstu_bwd_dkv_kernel<bf16_tag, D, false, false, 5>, WIN}
// (the three query-tile launches of a head dim above 256, on the kernels of the slot 256)
#define HSTU_BWD_WINDOWS(RAB, MASK)                                                                   \
    hstu_bwd_dq_kernel<bf16_tag, 256, RAB, MASK, 0, 1>, hstu_bwd_dq_kernel<bf16_tag, 256, RAB, MASK, 2, 2>, \
        hstu_bwd_dq_kernel<bf16_tag, 256, false, false, 0, 3>
#define HSTU_BWD_NO_WINDOWS nullptr, nullptr, nullptr
#define HSTU_BWD_DIMS(RAB, MASK)                                                                                     \
    {HSTU_BWD_VARIANT(64, RAB, MASK, HSTU_BWD_NO_WINDOWS), HSTU_BWD_VARIANT(128, RAB, MASK, HSTU_BWD_NO_WINDOWS), \
     HSTU_BWD_VARIANT(256, RAB, MASK, HSTU_BWD_WINDOWS(RAB, MASK))}
const BwdVariant kTable[2][2][3] = {{HSTU_BWD_DIMS(false, false), HSTU_BWD_DIMS(false, true)},
                                    {HSTU_BWD_DIMS(true, false), HSTU_BWD_DIMS(true, true)}};
}  // namespace
const BwdVariant (*bwd_variants_bf16())[2][3] { return kTable; }
}  // namespace hstu
