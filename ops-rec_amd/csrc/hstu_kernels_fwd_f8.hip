// forward kernels for fp8-e4m3 inputs
#include "hstu_variant_tables.h"

#define HSTU_F8_VARIANT(otag, oname, D, WGS)                                                    \
    {"hstu_fwd_f8e4m3_" oname "_d" #D, "hstu_fwd_f8e4m3_" oname "_d" #D "_queues",             \
     "hstu_fwd_f8e4m3_" oname "_d" #D "_split",                                                 \
     hstu::hstu_fwd_kernel<hstu::f8_tag, hstu::otag, D, false, false>,                          \
     hstu::queues_kernel<hstu::f8_tag, hstu::otag, D, false, false>(),                          \
     hstu::split_kernel<hstu::f8_tag, hstu::otag, D, false, false>(), nullptr, D, 256, WGS}

namespace hstu {
namespace {
const Variant kTable[2][3] = {
    {HSTU_F8_VARIANT(f16_tag, "f16", 64, 2), HSTU_F8_VARIANT(f16_tag, "f16", 128, 2), HSTU_F8_VARIANT(f16_tag, "f16", 256, 1)},
    {HSTU_F8_VARIANT(bf16_tag, "bf16", 64, 2), HSTU_F8_VARIANT(bf16_tag, "bf16", 128, 2),
     HSTU_F8_VARIANT(bf16_tag, "bf16", 256, 1)},
};
}
const Variant (*fwd_variants_f8())[3] { return kTable; }
}  // namespace hstu
