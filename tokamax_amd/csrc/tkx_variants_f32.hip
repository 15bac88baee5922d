// f32 x f32 kernel variants (true-f32 MFMA, forward, dlhs, drhs).
#include "tkx_gemm.hip.h"

namespace tkx {
#define FWD_DLHS(BM, BN, BK, WM, WN) \
  TKX_VARIANT(kFwd, kEF32, kEF32, BM, BN, BK, WM, WN), TKX_VARIANT(kDlhs, kEF32, kEF32, BM, BN, BK, WM, WN)

static const Variant kVariants[] = {
    FWD_DLHS(128, 128, 32, 2, 2),
    FWD_DLHS(64, 128, 32, 2, 2),
    FWD_DLHS(32, 128, 32, 1, 4),
    TKX_VARIANT(kDrhs, kEF32, kEF32, 128, 128, 32, 2, 2),
    TKX_VARIANT(kDrhs, kEF32, kEF32, 64, 128, 32, 2, 2),
};

const Variant* variants_f32(int* count) {
  *count = (int)(sizeof(kVariants) / sizeof(kVariants[0]));
  return kVariants;
}
}  // namespace tkx
