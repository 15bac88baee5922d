// bf16 activations x int8 weights forward variants (weights converted to bf16 on the way from LDS
// to the MFMA; per-(group, column) scales in the epilogue).
#include "tkx_gemm.hip.h"

namespace tkx {
static const Variant kVariants[] = {
    TKX_VARIANT(kFwd, kEBF16, kEI8, 128, 128, 64, 2, 2),
    TKX_VARIANT(kFwd, kEBF16, kEI8, 64, 128, 64, 2, 2),
    TKX_VARIANT(kFwd, kEBF16, kEI8, 32, 128, 64, 1, 4),
    TKX_VARIANT(kFwd, kEBF16, kEI8, 32, 256, 64, 1, 4),
    TKX_VARIANT(kFwd, kEBF16, kEI8, 32, 128, 128, 1, 4),
};

const Variant* variants_i8w(int* count) {
  *count = (int)(sizeof(kVariants) / sizeof(kVariants[0]));
  return kVariants;
}
}  // namespace tkx
