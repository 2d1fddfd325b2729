// forward kernels for bf16 inputs
#include "hstu_variant_tables.h"

namespace hstu {
namespace {
const Variant kTable[2][2][4] = HSTU_FWD16_TABLE(bf16_tag, "bf16");
}
const Variant (*fwd_variants_bf16())[2][4] { return kTable; }
}  // namespace hstu
