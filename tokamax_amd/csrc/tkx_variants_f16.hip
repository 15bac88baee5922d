// f16 x f16 kernel variants (forward, dlhs, drhs).
#include "tkx_gemm.hip.h"

namespace tkx {
#define FWD_DLHS(BM, BN, BK, WM, WN) \
  TKX_VARIANT(kFwd, kEF16, kEF16, BM, BN, BK, WM, WN), TKX_VARIANT(kDlhs, kEF16, kEF16, BM, BN, BK, WM, WN)

static const Variant kVariants[] = {
    FWD_DLHS(256, 256, 64, 2, 2),
    FWD_DLHS(128, 128, 64, 2, 2),
    FWD_DLHS(32, 128, 64, 1, 4),
    TKX_VARIANT(kDrhs, kEF16, kEF16, 128, 128, 64, 2, 2),
};

const Variant* variants_f16(int* count) {
  *count = (int)(sizeof(kVariants) / sizeof(kVariants[0]));
  return kVariants;
}
}  // namespace tkx
