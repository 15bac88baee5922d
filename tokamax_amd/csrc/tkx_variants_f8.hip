// OCP fp8 (e4m3fn) x fp8 forward variants; per-row / per-(group, column) scales in the epilogue.
#include "tkx_gemm.hip.h"

namespace tkx {
static const Variant kVariants[] = {
    TKX_VARIANT(kFwd, kEF8, kEF8, 256, 256, 128, 2, 2),
    TKX_VARIANT(kFwd, kEF8, kEF8, 256, 256, 128, 2, 4),
    TKX_VARIANT(kFwd, kEF8, kEF8, 128, 256, 128, 2, 2),
    TKX_VARIANT(kFwd, kEF8, kEF8, 128, 128, 128, 2, 2),
    TKX_VARIANT(kFwd, kEF8, kEF8, 64, 128, 128, 2, 2),
    TKX_VARIANT(kFwd, kEF8, kEF8, 32, 128, 128, 1, 4),
};

const Variant* variants_f8(int* count) {
  *count = (int)(sizeof(kVariants) / sizeof(kVariants[0]));
  return kVariants;
}
}  // namespace tkx
