// f16 x f16 kernel variants (forward, dlhs, drhs).
#include "tkx_gemm.hip.h"

namespace tkx {
#define FWD_DLHS(BM, BN, BK, WM, WN, NS) \
  TKX_VARIANT(kFwd, kEF16, kEF16, BM, BN, BK, WM, WN, NS), TKX_VARIANT(kDlhs, kEF16, kEF16, BM, BN, BK, WM, WN, NS)
#define DRHS(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kDrhs, kEF16, kEF16, BM, BN, BK, WM, WN, NS)

static const Variant kVariants[] = {
    TKX_VARIANT_SPLIT(kFwd, kEF16, kEF16, 256, 256, 64, 2, 4, 3, 4),  // A stages of 64 (whole lines), B stages of 32
    FWD_DLHS(256, 256, 32, 2, 4, 4),
    FWD_DLHS(128, 256, 64, 2, 4, 3),
    FWD_DLHS(128, 128, 64, 2, 2, 4),
    FWD_DLHS(32, 128, 64, 1, 4, 4),
    DRHS(128, 128, 64, 2, 2, 4),
    DRHS(256, 128, 32, 2, 2, 3),
    DRHS(256, 256, 32, 2, 4, 4),
};

const Variant* variants_f16(int* count) {
  *count = (int)(sizeof(kVariants) / sizeof(kVariants[0]));
  return kVariants;
}
}  // namespace tkx
