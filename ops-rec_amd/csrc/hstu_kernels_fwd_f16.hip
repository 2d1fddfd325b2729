// forward kernels for fp16 inputs
#include "hstu_variant_tables.h"

namespace hstu {
namespace {
const Variant kTable[2][2][4] = HSTU_FWD16_TABLE(f16_tag, "f16");
}
const Variant (*fwd_variants_f16())[2][4] { return kTable; }
}  // namespace hstu
