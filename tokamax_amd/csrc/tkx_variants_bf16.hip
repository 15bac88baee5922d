// bf16 x bf16 kernel variants (forward, dlhs, drhs).
#include "tkx_gemm.hip.h"

namespace tkx {
#define FWD_DLHS(BM, BN, BK, WM, WN, NS) \
  TKX_VARIANT(kFwd, kEBF16, kEBF16, BM, BN, BK, WM, WN, NS), TKX_VARIANT(kDlhs, kEBF16, kEBF16, BM, BN, BK, WM, WN, NS)
#define GLU(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kFwdGlu, kEBF16, kEBF16, BM, BN, BK, WM, WN, NS)
#define DRHS(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kDrhs, kEBF16, kEBF16, BM, BN, BK, WM, WN, NS)

static const Variant kVariants[] = {
    // split pipeline: A stages of 64 (whole 128-byte lines), B stages of 32; (A stages, B stages) = (3, 4): 160 KB
    TKX_VARIANT_SPLIT(kFwd, kEBF16, kEBF16, 256, 256, 64, 2, 4, 3, 4),
    FWD_DLHS(256, 256, 64, 2, 4, 2),
    FWD_DLHS(256, 256, 32, 2, 4, 4),
    FWD_DLHS(256, 256, 32, 2, 4, 5),
    FWD_DLHS(256, 128, 64, 2, 4, 3),
    FWD_DLHS(128, 256, 64, 2, 4, 3),
    FWD_DLHS(128, 256, 64, 2, 2, 3),
    FWD_DLHS(128, 256, 32, 2, 4, 5),
    FWD_DLHS(128, 256, 32, 2, 2, 3),
    FWD_DLHS(128, 128, 64, 2, 2, 4),
    FWD_DLHS(128, 128, 64, 2, 2, 2),
    FWD_DLHS(64, 256, 64, 2, 2, 3),
    FWD_DLHS(64, 128, 64, 2, 2, 4),
    FWD_DLHS(32, 256, 64, 1, 4, 3),
    FWD_DLHS(32, 128, 64, 1, 4, 4),
    GLU(256, 256, 32, 2, 4, 4),
    GLU(256, 256, 64, 2, 4, 2),
    GLU(128, 256, 64, 2, 4, 3),
    GLU(64, 256, 64, 2, 2, 3),
    GLU(32, 256, 64, 1, 4, 3),
    DRHS(256, 256, 64, 2, 4, 2),
    DRHS(256, 256, 32, 2, 4, 4),
    DRHS(128, 256, 64, 2, 4, 3),
    DRHS(128, 256, 32, 2, 2, 3),
    DRHS(256, 128, 32, 2, 2, 3),
    DRHS(128, 128, 64, 2, 2, 4),
    DRHS(64, 128, 64, 2, 2, 4),
};

const Variant* variants_bf16(int* count) {
  *count = (int)(sizeof(kVariants) / sizeof(kVariants[0]));
  return kVariants;
}
}  // namespace tkx
