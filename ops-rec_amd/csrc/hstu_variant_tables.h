// Builders of the variant tables; included by the translation units that instantiate forward kernels.
#pragma once
#include "hstu_fwd_kernel.hip.h"
#include "hstu_variants.h"

namespace hstu {

template <typename Tag, typename OutTag, int D, bool RAB, bool MASK>
constexpr auto queues_kernel() -> void (*)(const FwdArgs)
{
    // (at the slot 32, four workgroups per CU and the fewest flops per byte streamed: plain list -> queues 128 x 8 heads of
    // 4096 rows 2.96 -> 2.19 ms, 512 x 8 of 1024 rows 933 -> 760 us, 1024 x 4 of 256..1024 rows 506 -> 399 us)
    // (at the slot 256, one workgroup per CU: plain list -> queues 32 x 8 heads of 4096 rows 3.12 -> 2.47 ms, 64 x 4 of
    // 1024..4096 rows 1.43 -> 1.23 ms, 256 x 4 of 256..1024 rows 575 -> 502 us, 32 x 4 of 512..2048 rows 199 -> 188 us)
    if constexpr (D == 32 || D == 64 || D == 128 || D == 256) {
        return hstu_fwd_kernel<Tag, OutTag, D, RAB, MASK, true>;
    } else {
        return nullptr;
    }
}

template <typename Tag, typename OutTag, int D, bool RAB, bool MASK>
constexpr auto split_kernel() -> void (*)(const FwdArgs)
{
    // (at the slot 256 split items were measured level with the plain list: -12 .. +16 % over ten shapes)
    if constexpr (D == 64 || D == 128) {
        return hstu_fwd_kernel<Tag, OutTag, D, RAB, MASK, false, true>;
    } else {
        return nullptr;
    }
}

template <typename Tag, typename OutTag, int D, bool RAB, bool MASK>
constexpr auto paged_kernel() -> void (*)(const FwdArgs)
{
    if constexpr (D == 64 || D == 128 || D == 256) {
        return hstu_fwd_kernel<Tag, OutTag, D, RAB, MASK, false, true, true>;
    } else {
        return nullptr;
    }
}

}  // namespace hstu

#define HSTU_VARIANT(tag, tagname, D, RAB, MASK)                                              \
    {"hstu_fwd_" tagname "_d" #D "_rab" #RAB "_mask" #MASK,                                        \
     "hstu_fwd_" tagname "_d" #D "_rab" #RAB "_mask" #MASK "_queues",                               \
     "hstu_fwd_" tagname "_d" #D "_rab" #RAB "_mask" #MASK "_split",                                \
     hstu::hstu_fwd_kernel<hstu::tag, hstu::tag, D, RAB, MASK>,                                     \
     hstu::queues_kernel<hstu::tag, hstu::tag, D, RAB, MASK>(),                                     \
     hstu::split_kernel<hstu::tag, hstu::tag, D, RAB, MASK>(),                                      \
     hstu::paged_kernel<hstu::tag, hstu::tag, D, RAB, MASK>(), D, 256, hstu::fwd_wgs_per_cu(D, RAB, MASK)}
#define HSTU_DIMS(tag, tagname, RAB, MASK)                                                           \
    {HSTU_VARIANT(tag, tagname, 32, RAB, MASK), HSTU_VARIANT(tag, tagname, 64, RAB, MASK), \
     HSTU_VARIANT(tag, tagname, 128, RAB, MASK), HSTU_VARIANT(tag, tagname, 256, RAB, MASK)}
// one 16-bit input type: [rab][custom mask][dim slot]
#define HSTU_FWD16_TABLE(tag, tagname)                                         \
    {{HSTU_DIMS(tag, tagname, false, false), HSTU_DIMS(tag, tagname, false, true)}, \
     {HSTU_DIMS(tag, tagname, true, false), HSTU_DIMS(tag, tagname, true, true)}}
