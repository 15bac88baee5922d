// f32 x f32 kernel variants (true-f32 MFMA; forward, dlhs, drhs).
#include "tkx_gemm.hip.h"

namespace tkx {
#define FWD_DLHS(BM, BN, BK, WM, WN, NS) \
  TKX_VARIANT(kFwd, kEF32, kEF32, BM, BN, BK, WM, WN, NS), TKX_VARIANT(kDlhs, kEF32, kEF32, BM, BN, BK, WM, WN, NS)
#define DRHS(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kDrhs, kEF32, kEF32, BM, BN, BK, WM, WN, NS)

static const Variant kVariants[] = {
    FWD_DLHS(128, 128, 32, 2, 2, 4),
    FWD_DLHS(64, 128, 32, 2, 2, 4),
    FWD_DLHS(32, 128, 32, 1, 4, 4),
    DRHS(128, 128, 32, 2, 2, 4),
    DRHS(64, 128, 32, 2, 2, 4),
};

const Variant* variants_f32(int* count) {
  *count = (int)(sizeof(kVariants) / sizeof(kVariants[0]));
  return kVariants;
}
}  // namespace tkx
