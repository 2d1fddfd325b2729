// forward kernels for fp8-e4m3 inputs
#include "hstu_variant_tables.h"

// without rab / custom mask: plain, queue and split variants
#define HSTU_F8_VARIANT(otag, oname, D, WGS)                                                    \
    {"hstu_fwd_f8e4m3_" oname "_d" #D, "hstu_fwd_f8e4m3_" oname "_d" #D "_queues",             \
     "hstu_fwd_f8e4m3_" oname "_d" #D "_split",                                                 \
     hstu::hstu_fwd_kernel<hstu::f8_tag, hstu::otag, D, false, false>,                          \
     hstu::queues_kernel<hstu::f8_tag, hstu::otag, D, false, false>(),                          \
     hstu::split_kernel<hstu::f8_tag, hstu::otag, D, false, false>(), nullptr, D, 256, hstu::fwd_wgs_per_cu(D, false, false)}
// with rab and / or a custom mask (e4m3 tensors like q): the plain list, and the per-XCD queues for long lists
#define HSTU_F8_BIASED(otag, oname, D, RAB, MASK, WGS)                                          \
    {"hstu_fwd_f8e4m3_" oname "_d" #D "_rab" #RAB "_mask" #MASK,                                \
     "hstu_fwd_f8e4m3_" oname "_d" #D "_rab" #RAB "_mask" #MASK "_queues", nullptr,             \
     hstu::hstu_fwd_kernel<hstu::f8_tag, hstu::otag, D, RAB, MASK>,                             \
     hstu::queues_kernel<hstu::f8_tag, hstu::otag, D, RAB, MASK>(), nullptr, nullptr, D, 256, hstu::fwd_wgs_per_cu(D, RAB, MASK)}
#define HSTU_F8_DIMS(otag, oname)                                                                \
    {{{HSTU_F8_VARIANT(otag, oname, 64, 2), HSTU_F8_VARIANT(otag, oname, 128, 2), HSTU_F8_VARIANT(otag, oname, 256, 1)},   \
      {HSTU_F8_BIASED(otag, oname, 64, false, true, 2), HSTU_F8_BIASED(otag, oname, 128, false, true, 2),                  \
       HSTU_F8_BIASED(otag, oname, 256, false, true, 1)}},                                                                 \
     {{HSTU_F8_BIASED(otag, oname, 64, true, false, 2), HSTU_F8_BIASED(otag, oname, 128, true, false, 2),                  \
       HSTU_F8_BIASED(otag, oname, 256, true, false, 1)},                                                                  \
      {HSTU_F8_BIASED(otag, oname, 64, true, true, 2), HSTU_F8_BIASED(otag, oname, 128, true, true, 2),                    \
       HSTU_F8_BIASED(otag, oname, 256, true, true, 1)}}}

namespace hstu {
namespace {
// [output: fp16, bf16][rab][custom mask][dim slot: 64, 128, 256]
const Variant kTable[2][2][2][3] = {HSTU_F8_DIMS(f16_tag, "f16"), HSTU_F8_DIMS(bf16_tag, "bf16")};
}
const Variant (*fwd_variants_f8())[2][2][3] { return kTable; }
}  // namespace hstu
