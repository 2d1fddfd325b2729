// kernels for short work lists / short rows (16-bit inputs, head-dim slot 128, no custom mask): the forward (with and
// without attn_bias), the forward and the backward for batches of tiny sequences, the backward for sequences of few query
// rows, and the backward's query-tile kernel (no bias)
#include "hstu_bwd_dq_short_kernel.hip.h"
#include "hstu_bwd_few_rows_kernel.hip.h"
#include "hstu_bwd_tiny_kernel.hip.h"
#include "hstu_fwd_few_rows_kernel.hip.h"
#include "hstu_fwd_short_kernel.hip.h"
#include "hstu_fwd_tiny_kernel.hip.h"
#include "hstu_variants.h"

namespace hstu {
namespace {
const ShortVariant kTable[4] = {
    {"hstu_fwd_bf16_d128_short", hstu_fwd_short_kernel<bf16_tag, 128>},
    {"hstu_fwd_f16_d128_short", hstu_fwd_short_kernel<f16_tag, 128>},
    {"hstu_fwd_bf16_d128_rab_short", hstu_fwd_short_kernel<bf16_tag, 128, true>},
    {"hstu_fwd_f16_d128_rab_short", hstu_fwd_short_kernel<f16_tag, 128, true>},
};
}
const ShortVariant* fwd_variants_short() { return kTable; }

namespace {
#define HSTU_TINY(tag, tagname, D, R) {"hstu_fwd_" tagname "_d" #D "_tiny" #R, hstu_fwd_tiny_kernel<tag, D, R>}
const ShortVariant kTiny[2][3][2] = {
    {{HSTU_TINY(bf16_tag, "bf16", 64, 32), HSTU_TINY(bf16_tag, "bf16", 64, 64)},
     {HSTU_TINY(bf16_tag, "bf16", 128, 32), HSTU_TINY(bf16_tag, "bf16", 128, 64)},
     {HSTU_TINY(bf16_tag, "bf16", 256, 32), HSTU_TINY(bf16_tag, "bf16", 256, 64)}},
    {{HSTU_TINY(f16_tag, "f16", 64, 32), HSTU_TINY(f16_tag, "f16", 64, 64)},
     {HSTU_TINY(f16_tag, "f16", 128, 32), HSTU_TINY(f16_tag, "f16", 128, 64)},
     {HSTU_TINY(f16_tag, "f16", 256, 32), HSTU_TINY(f16_tag, "f16", 256, 64)}},
};
}
const ShortVariant (*fwd_variants_tiny())[3][2] { return kTiny; }

namespace {
const ShortVariant kFwdFewRows[2][2] = {
    {{"hstu_fwd_bf16_d64_few_rows", hstu_fwd_few_rows_kernel<bf16_tag, 64>}, {"hstu_fwd_bf16_d128_few_rows", hstu_fwd_few_rows_kernel<bf16_tag, 128>}},
    {{"hstu_fwd_f16_d64_few_rows", hstu_fwd_few_rows_kernel<f16_tag, 64>}, {"hstu_fwd_f16_d128_few_rows", hstu_fwd_few_rows_kernel<f16_tag, 128>}},
};
}
const ShortVariant (*fwd_variants_few_rows())[2] { return kFwdFewRows; }

namespace {
const DqShortVariant kDqShort[2] = {
    {hstu_bwd_dq_short_kernel<bf16_tag, 128, 0>, hstu_bwd_dq_short_kernel<bf16_tag, 128, 1>, hstu_bwd_dq_short_kernel<bf16_tag, 128, 2>},
    {hstu_bwd_dq_short_kernel<f16_tag, 128, 0>, hstu_bwd_dq_short_kernel<f16_tag, 128, 1>, hstu_bwd_dq_short_kernel<f16_tag, 128, 2>},
};
}
const DqShortVariant* bwd_variants_dq_short() { return kDqShort; }

namespace {
const BwdTinyVariant kBwdTiny[2][2] = {
    {{"hstu_bwd_bf16_d128_tiny", hstu_bwd_tiny_kernel<bf16_tag, 128>}, {"hstu_bwd_bf16_d256_tiny", hstu_bwd_tiny_kernel<bf16_tag, 256>}},
    {{"hstu_bwd_f16_d128_tiny", hstu_bwd_tiny_kernel<f16_tag, 128>}, {"hstu_bwd_f16_d256_tiny", hstu_bwd_tiny_kernel<f16_tag, 256>}},
};
}
const BwdTinyVariant (*bwd_variants_tiny())[2] { return kBwdTiny; }

namespace {
const BwdTinyVariant kBwdFewRows[2][2] = {
    {{"hstu_bwd_bf16_d64_few_rows", hstu_bwd_few_rows_kernel<bf16_tag, 64>}, {"hstu_bwd_bf16_d128_few_rows", hstu_bwd_few_rows_kernel<bf16_tag, 128>}},
    {{"hstu_bwd_f16_d64_few_rows", hstu_bwd_few_rows_kernel<f16_tag, 64>}, {"hstu_bwd_f16_d128_few_rows", hstu_bwd_few_rows_kernel<f16_tag, 128>}},
};
}
const BwdTinyVariant (*bwd_variants_few_rows())[2] { return kBwdFewRows; }
}  // namespace hstu
